// Block dequantization to float32, one "unit" of a block per thread, shared by the
// verification export and the embedding lookup.  A unit is the slice of a block that one
// aligned dword (or dword pair) of quants expands to; emit(k, value) receives the element
// index inside the block and the value.
//   Q4_K  32 units of 8 values  (gguf.py:631-643)
//   Q5_K  32 units of 8 values  (gguf.py:646-662)
//   Q6_K  16 units of 16 values (gguf.py:665-681)
//   Q8_0   8 units of 4 values  (gguf.py:604-608)
#pragma once

#include "gguf_common.hpp"

namespace hipengine_gfx950 {

template <int QT>
struct DequantTraits;
template <> struct DequantTraits<GGML_Q4_K> { static constexpr int BYTES = Q4_K_BYTES, VALUES = QK_K, UNITS = 32; };
template <> struct DequantTraits<GGML_Q5_K> { static constexpr int BYTES = Q5_K_BYTES, VALUES = QK_K, UNITS = 32; };
template <> struct DequantTraits<GGML_Q6_K> { static constexpr int BYTES = Q6_K_BYTES, VALUES = QK_K, UNITS = 16; };
template <> struct DequantTraits<GGML_Q8_0> { static constexpr int BYTES = Q8_0_BYTES, VALUES = 32, UNITS = 8; };

__device__ __forceinline__ float dq_byte_f(uint32_t w, int i) { return static_cast<float>((w >> (8 * i)) & 0xFFu); }

template <int QT, class Emit>
__device__ __forceinline__ void dequant_unit(const uint8_t* blk, int i, Emit emit) {
  if constexpr (QT == GGML_Q4_K || QT == GGML_Q5_K) {
    // unit i = dword i of qs: sub-block pair i/8, lanes 4*(i%8)..+3; low nibbles are sub-block
    // 2*pair, high nibbles 2*pair+1
    constexpr int QS = QT == GGML_Q4_K ? 16 : 48;
    const uint4 h = load16(blk);
    const uint32_t qs = load4(blk + QS + 4 * i);
    const Q4KScales s = q4k_unpack_scales(h.y, h.z, h.w);
    const float d = f16_bits_to_float(h.x & 0xFFFFu), dmin = f16_bits_to_float(h.x >> 16);
    const int pair = i >> 3, lane0 = (i & 7) * 4;
    const float sa = d * static_cast<float>(q4k_scale_of(s, 2 * pair));
    const float sb = d * static_cast<float>(q4k_scale_of(s, 2 * pair + 1));
    const float ma = dmin * static_cast<float>(q4k_min_of(s, 2 * pair));
    const float mb = dmin * static_cast<float>(q4k_min_of(s, 2 * pair + 1));
    uint32_t lo = q4k_low(qs), hi = q4k_high(qs);
    if constexpr (QT == GGML_Q5_K) {
      // bit 4 of the value of sub-block s, lane l is bit s of qh[l]
      const uint32_t qh = load4(blk + 16 + lane0);
      lo |= ((qh >> (2 * pair)) & 0x01010101u) << 4;
      hi |= ((qh >> (2 * pair + 1)) & 0x01010101u) << 4;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      emit((2 * pair) * 32 + lane0 + j, sa * dq_byte_f(lo, j) - ma);
      emit((2 * pair + 1) * 32 + lane0 + j, sb * dq_byte_f(hi, j) - mb);
    }
  } else if constexpr (QT == GGML_Q6_K) {
    // unit = (half h, lane dword i): four groups of 32 share the dword position
    const int h = i >> 3, l = i & 7;
    const Q6KQuad u = q6k_unpack(load4(blk + 64 * h + 4 * l), load4(blk + 64 * h + 32 + 4 * l),
                                 load4(blk + 128 + 32 * h + 4 * l));
    const uint32_t g[4] = {q6k_center(u.g0), q6k_center(u.g1), q6k_center(u.g2), q6k_center(u.g3)};
    const float d = f16_bits_to_float(load2(blk + 208));
    const int8_t* sc = reinterpret_cast<const int8_t*>(blk + 192);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int grp = 4 * h + j;
      const float step = d * static_cast<float>(sc[grp * 2 + (l >> 2)]);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int q = static_cast<int8_t>((g[j] >> (8 * e)) & 0xFFu);
        emit(grp * 32 + 4 * l + e, step * static_cast<float>(q));
      }
    }
  } else {
    const float d = f16_bits_to_float(load2(blk));
    const uint32_t w = (load2(blk + 2 + 4 * i)) | (load2(blk + 4 + 4 * i) << 16);
#pragma unroll
    for (int e = 0; e < 4; ++e) emit(4 * i + e, static_cast<float>(static_cast<int8_t>((w >> (8 * e)) & 0xFFu)) * d);
  }
}

}  // namespace hipengine_gfx950
