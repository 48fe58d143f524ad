// Shared device helpers for the gfx950 GGUF k-quant kernels: block geometry,
// fp16/bf16 conversion, wave64 DPP reductions and the integer unpack of
// Q4_K / Q6_K / Q8_0 blocks into packed int8 dwords.
//
// Every kernel in this directory (GEMV, MMQ, MoE, the dequantize and
// block-dot verification exports) unpacks weights through the functions in
// this header, so a bit-exact check of the verification exports is a check of
// the unpack the production kernels execute.
//
// Block layouts (little endian), as hipEngine stores them
// (hipengine/quant/gguf.py:171-210):
//   Q4_K 144 B / 256 values: half d; half dmin; u8 scales[12]; u8 qs[128]
//   Q6_K 210 B / 256 values: u8 ql[128]; u8 qh[64]; i8 scales[16]; half d
//   Q8_0  34 B /  32 values: half d; i8 qs[32]
//   q8_1  36 B /  32 values: half d; half s; i8 qs[32]
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace hipengine_gfx950 {

using half_t = _Float16;

constexpr int QK_K = 256;
constexpr int Q4_K_BYTES = 144;
constexpr int Q5_K_BYTES = 176;
constexpr int Q6_K_BYTES = 210;
constexpr int Q8_0_BYTES = 34;
constexpr int Q8_1_BYTES = 36;
constexpr int DS4_BYTES = 144;
constexpr int D4S4_BYTES = 160;

// GGML type ids (hipengine/quant/gguf.py:23-57)
constexpr int GGML_Q8_0 = 8;
constexpr int GGML_Q4_K = 12;
constexpr int GGML_Q5_K = 13;
constexpr int GGML_Q6_K = 14;

// Element types at the C boundary.
enum ScalarKind : int { KIND_F32 = 0, KIND_BF16 = 1, KIND_F16 = 2, KIND_Q8_1 = 3 };

__device__ __forceinline__ float bits_to_float(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t float_to_bits(float f) { return __builtin_bit_cast(uint32_t, f); }

__device__ __forceinline__ float f16_bits_to_float(uint32_t lo16) {
  return static_cast<float>(__builtin_bit_cast(half_t, static_cast<uint16_t>(lo16)));
}

__device__ __forceinline__ uint16_t float_to_f16_bits(float v) {
  return __builtin_bit_cast(uint16_t, static_cast<half_t>(v));
}

__device__ __forceinline__ float bf16_bits_to_float(uint32_t lo16) { return bits_to_float(lo16 << 16); }

// Round to nearest even by "+0x7FFF+lsb", no NaN special case
// (kernels/hip_gfx1100/quant/gguf_q4_k_gemv.hip:32-41).
__device__ __forceinline__ uint16_t float_to_bf16_bits(float v) {
  uint32_t u = float_to_bits(v);
  u += 0x7FFFu + ((u >> 16) & 1u);
  return static_cast<uint16_t>(u >> 16);
}

__device__ __forceinline__ void store_scalar(void* out, int64_t idx, float v, int kind) {
  if (kind == KIND_F32) {
    static_cast<float*>(out)[idx] = v;
  } else if (kind == KIND_BF16) {
    static_cast<uint16_t*>(out)[idx] = float_to_bf16_bits(v);
  } else {
    static_cast<uint16_t*>(out)[idx] = float_to_f16_bits(v);
  }
}

__device__ __forceinline__ float load_scalar(const void* x, int64_t idx, int kind) {
  if (kind == KIND_F32) return static_cast<const float*>(x)[idx];
  const uint32_t b = static_cast<const uint16_t*>(x)[idx];
  return kind == KIND_BF16 ? bf16_bits_to_float(b) : f16_bits_to_float(b);
}

// ---- wave64 cross-lane helpers (DPP; no LDS) -----------------------------

// Round-trip through the output type (what a separate kernel reading the stored value would see).
__device__ __forceinline__ float round_to_kind(float v, int kind) {
  if (kind == KIND_BF16) return bf16_bits_to_float(float_to_bf16_bits(v));
  if (kind == KIND_F16) return f16_bits_to_float(float_to_f16_bits(v));
  return v;
}

template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
template <int CTRL>
__device__ __forceinline__ int dpp_i(int v) {
  return __builtin_amdgcn_mov_dpp(v, CTRL, 0xF, 0xF, true);
}

constexpr int DPP_QUAD_XOR1 = 0xB1;     // quad_perm:[1,0,3,2]
constexpr int DPP_QUAD_XOR2 = 0x4E;     // quad_perm:[2,3,0,1]
constexpr int DPP_ROW_HALF_MIRROR = 0x141;  // lane i <-> lane 7-i inside each group of 8
constexpr int DPP_ROW_SHL1 = 0x101;     // lane i reads lane i+1 (inside a row of 16)
constexpr int DPP_ROW_SHL2 = 0x102;
constexpr int DPP_ROW_SHL4 = 0x104;

// All four lanes of a quad receive the quad total.
__device__ __forceinline__ float quad_sum(float v) {
  v += dpp_f<DPP_QUAD_XOR1>(v);
  v += dpp_f<DPP_QUAD_XOR2>(v);
  return v;
}

// All eight lanes of an aligned group of 8 receive the group maximum.
// Maximum over an aligned group of 8 lanes of a NON-NEGATIVE float: the bit patterns of
// non-negative floats order like unsigned integers, and the integer maximum takes its DPP
// operand directly (one instruction per stage, no NaN canonicalization).
__device__ __forceinline__ float oct_max(float v) {
  uint32_t u = float_to_bits(v);
  u = max(u, static_cast<uint32_t>(dpp_i<DPP_QUAD_XOR1>(static_cast<int>(u))));
  u = max(u, static_cast<uint32_t>(dpp_i<DPP_QUAD_XOR2>(static_cast<int>(u))));
  u = max(u, static_cast<uint32_t>(dpp_i<DPP_ROW_HALF_MIRROR>(static_cast<int>(u))));
  return bits_to_float(u);
}

__device__ __forceinline__ int oct_sum_i(int v) {
  v += dpp_i<DPP_QUAD_XOR1>(v);
  v += dpp_i<DPP_QUAD_XOR2>(v);
  v += dpp_i<DPP_ROW_HALF_MIRROR>(v);
  return v;
}

// Sum of 32 floats held four per lane by an aligned group of 8 lanes (lane t
// holds elements 4t..4t+3), added in the order of a 32-lane shfl_down tree:
// element i += element i+16, then +8, +4, +2, +1
// (kernels/hip_gfx1100/quant/gguf_q4_k_gemv.hip:130-135).  The result is valid
// in lane 0 of the group.
__device__ __forceinline__ float oct_tree_sum32(float a, float b, float c, float d) {
  a += dpp_f<DPP_ROW_SHL4>(a); b += dpp_f<DPP_ROW_SHL4>(b);   // i += i+16
  c += dpp_f<DPP_ROW_SHL4>(c); d += dpp_f<DPP_ROW_SHL4>(d);
  a += dpp_f<DPP_ROW_SHL2>(a); b += dpp_f<DPP_ROW_SHL2>(b);   // i += i+8
  c += dpp_f<DPP_ROW_SHL2>(c); d += dpp_f<DPP_ROW_SHL2>(d);
  a += dpp_f<DPP_ROW_SHL1>(a); b += dpp_f<DPP_ROW_SHL1>(b);   // i += i+4
  c += dpp_f<DPP_ROW_SHL1>(c); d += dpp_f<DPP_ROW_SHL1>(d);
  a += c;                                                      // i += i+2
  b += d;
  return a + b;                                                // i += i+1
}

// ---- integer dot --------------------------------------------------------

// Four signed int8 products accumulated into int32 (v_dot4_i32_i8).  Weights
// that are unsigned nibbles or 6-bit values (0..63) are valid signed bytes.
__device__ __forceinline__ int dot4(uint32_t w, uint32_t x, int acc) {
  return __builtin_amdgcn_sdot4(static_cast<int>(w), static_cast<int>(x), acc, false);
}

// ---- Q4_K ------------------------------------------------------------------

// The 12 scale bytes as three dwords -> four dwords holding the eight 6-bit
// scales and eight 6-bit mins, one per byte
// (hipengine/quant/gguf.py:611-624, gguf_q4_k_gemv.hip:74-88).
struct Q4KScales {
  uint32_t sc_lo, sc_hi, mn_lo, mn_hi;  // bytes j&3 of *_lo (j<4) / *_hi (j>=4)
};

__device__ __forceinline__ Q4KScales q4k_unpack_scales(uint32_t s0, uint32_t s1, uint32_t s2) {
  Q4KScales r;
  r.sc_lo = s0 & 0x3F3F3F3Fu;
  r.mn_lo = s1 & 0x3F3F3F3Fu;
  r.sc_hi = (s2 & 0x0F0F0F0Fu) | ((s0 >> 2) & 0x30303030u);
  r.mn_hi = ((s2 >> 4) & 0x0F0F0F0Fu) | ((s1 >> 2) & 0x30303030u);
  return r;
}

__device__ __forceinline__ uint32_t q4k_scale_of(const Q4KScales& s, int sb) {
  return ((sb < 4 ? s.sc_lo : s.sc_hi) >> (8 * (sb & 3))) & 0xFFu;
}
__device__ __forceinline__ uint32_t q4k_min_of(const Q4KScales& s, int sb) {
  return ((sb < 4 ? s.mn_lo : s.mn_hi) >> (8 * (sb & 3))) & 0xFFu;
}

// One dword of qs bytes (4 consecutive bytes of a 32-byte pair group) carries
// 4 values of sub-block 2p in the low nibbles and 4 of sub-block 2p+1 in the
// high nibbles (gguf_q4_k_gemv.hip:90-106).
__device__ __forceinline__ uint32_t q4k_low(uint32_t qs) { return qs & 0x0F0F0F0Fu; }
__device__ __forceinline__ uint32_t q4k_high(uint32_t qs) { return (qs >> 4) & 0x0F0F0F0Fu; }

// ---- Q6_K ------------------------------------------------------------------

// Four consecutive lanes' worth (one dword each) of ql and qh for one half
// (128 values) of a block: `qla` from ql[64h + lane..], `qlb` from
// ql[64h + 32 + lane..], `qh` from qh[32h + lane..].  Returns the unsigned
// 6-bit values (0..63) of groups 4h+0..4h+3 at those four lanes
// (hipengine/quant/gguf.py:665-681, gguf_k_gemv.hip:139-160).
struct Q6KQuad {
  uint32_t g0, g1, g2, g3;
};

__device__ __forceinline__ Q6KQuad q6k_unpack(uint32_t qla, uint32_t qlb, uint32_t qh) {
  Q6KQuad r;
  r.g0 = (qla & 0x0F0F0F0Fu) | ((qh << 4) & 0x30303030u);
  r.g1 = (qlb & 0x0F0F0F0Fu) | ((qh << 2) & 0x30303030u);
  r.g2 = ((qla >> 4) & 0x0F0F0F0Fu) | (qh & 0x30303030u);
  r.g3 = ((qlb >> 4) & 0x0F0F0F0Fu) | ((qh >> 2) & 0x30303030u);
  return r;
}

// Bytewise (u6 - 32) for four packed values 0..63: no byte borrows because
// (u | 0x80) - 0x20 stays within the byte, then the 0x80 marker is flipped back.
__device__ __forceinline__ uint32_t q6k_center(uint32_t u6x4) {
  return ((u6x4 | 0x80808080u) - 0x20202020u) ^ 0x80808080u;
}

// Loads from GGUF blocks, which are only 2-byte aligned (Q6_K 210 B, Q8_0 34 B).
__device__ __forceinline__ uint4 load16(const uint8_t* p) {
  uint4 v;
  __builtin_memcpy(&v, __builtin_assume_aligned(p, 2), 16);
  return v;
}
__device__ __forceinline__ uint2 load8(const uint8_t* p) {
  uint2 v;
  __builtin_memcpy(&v, __builtin_assume_aligned(p, 2), 8);
  return v;
}
__device__ __forceinline__ uint32_t load4(const uint8_t* p) {
  uint32_t v;
  __builtin_memcpy(&v, __builtin_assume_aligned(p, 2), 4);
  return v;
}
__device__ __forceinline__ uint32_t load2(const uint8_t* p) {
  uint16_t v;
  __builtin_memcpy(&v, __builtin_assume_aligned(p, 2), 2);
  return v;
}

// ---- loads from global memory straight into LDS --------------------------------------------
//
// global_load_lds_dwordx4 / _dword: lane l's 16 (4) bytes at `base + voff` land at LDS byte `lds` + 16 l (4 l);
// no register holds the data while the load is in flight.  The compiler does not see these as memory
// operations with a result: completion is waited for with s_waitcnt vmcnt (loads complete in issue order),
// by hand or through the wait the compiler places for a load of its own that was issued later.
typedef __attribute__((address_space(3))) uint8_t lds_u8;

__device__ __forceinline__ uint32_t lds_address(const void* p) {
  return static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_u8*)p));
}
__device__ __forceinline__ void lds_dma16(const uint8_t* base, uint32_t voff, uint32_t lds) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds), "v"(voff), "s"(base) : "memory");
}
__device__ __forceinline__ void lds_dma4(const uint8_t* base, uint32_t voff, uint32_t lds) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" ::"s"(lds), "v"(voff), "s"(base) : "memory");
}

}  // namespace hipengine_gfx950
