// Decode GEMV for raw GGUF Q4_K / Q6_K / Q8_0 weights on gfx950, batch 1..8,
// with the q8_1 activation quantization fused in front.
//
//   out[b, n] = sum_k  W[n, k] * x[b, k]
//
// evaluated as int32 sub-block dots of the packed weight integers with int8
// activations (v_dot4_i32_i8), combined in float32 with the block scales:
//   Q4_K: xd*(d*sc*dot - dmin*mn*qsum)   (gguf_q4_k_gemv.hip:893-904)
//   Q5_K: the same with 5-bit quants       (gguf_k_gemv.hip:115-137)
//   Q6_K: xd*d*sc16*(dot_u - 32*qsum16)  (gguf_k_gemv.hip:233-246)
//   Q8_0: wd*xd*dot                      (gguf_q8_0_dp4a_gemv.hip:122-129)
//
// Work decomposition (wave64, 256 CUs):
//   * A workgroup owns `nrg*16*R` consecutive output rows.  Its waves form a
//     grid of `ks` K-slices by `nrg` row groups.
//   * Inside a wave, 4 adjacent lanes share one 256-value weight block: lane
//     q streams the bytes of 64 of its values (plus the block header) with
//     16-byte loads, so one load instruction of a wave covers 16 rows and all
//     bytes of a row are fetched exactly once.  Sixteen such lane quads cover
//     16 rows; R > 1 repeats the pattern 16 rows further down.
//   * The K range is walked in chunks of `ks*CB` blocks.  For each chunk every
//     wave first issues the loads of its CB blocks, then all waves of the
//     workgroup quantize the chunk's activations to q8_1 into LDS together
//     (8 lanes per 32 values), and only then consume them, so the HBM latency
//     of the weight stream overlaps the quantization.
//   * The four lanes of a block reduce with DPP; K-slices reduce through LDS.
//
// Activations are read from LDS as broadcast 16-byte reads (all 16 row lanes
// of a wave read the same address), weights never touch LDS.
#pragma once

#include "gguf_common.hpp"

namespace hipengine_gfx950 {

struct GemvArgs {
  const void* x;        // [rows, K] scalars of x_kind, or q8_1 blocks [rows, K/32] when KIND_Q8_1
  const uint8_t* w;     // [N, row_bytes] raw blocks (expert-indexed variants add an offset per row group)
  void* out;            // [rows, N] scalars of out_kind
  int x_kind;
  int out_kind;
  int rows;             // 1..B
  int K;
  int N;
  int ks;               // K-slices per workgroup
  int nrg;              // row groups per workgroup
  const void* x_up;     // KIND_SILU_BF16 only: the second bf16 operand, the activation is bf16(silu(x) * x_up)
};

// Activation kind of the expert-selected down projection that takes the gate and up rows as they are
// (bf16) and forms bf16(silu(gate) * up) while staging (gguf_k_gemv.hip:1813-1866).  Not part of the C ABI.
constexpr int KIND_SILU_BF16 = 4;

// Q4_K and Q5_K share the header (d, dmin, 6-bit scales and mins) and the min term.
constexpr bool gemv_has_mins(int qt) { return qt == GGML_Q4_K || qt == GGML_Q5_K; }

template <int QT>
struct GemvTraits;

template <>
struct GemvTraits<GGML_Q4_K> {
  static constexpr int SUPER_BYTES = Q4_K_BYTES;  // bytes per 256 values
  static constexpr int REGS = 12;
};
template <>
struct GemvTraits<GGML_Q5_K> {
  static constexpr int SUPER_BYTES = Q5_K_BYTES;
  static constexpr int REGS = 20;   // header 4, low nibbles 8, high bits qh[32] 8
};
template <>
struct GemvTraits<GGML_Q6_K> {
  static constexpr int SUPER_BYTES = Q6_K_BYTES;
  static constexpr int REGS = 15;
};
template <>
struct GemvTraits<GGML_Q8_0> {
  static constexpr int SUPER_BYTES = 8 * Q8_0_BYTES;  // eight 34-byte blocks
  static constexpr int REGS = 17;
};

template <int N>
struct WeightRegs {
  uint32_t v[N];
};

// Lane q (0..3) of a quad loads its share of the 256-value block at `blk`.
template <int QT>
__device__ __forceinline__ void gemv_load_block(const uint8_t* blk, int q, WeightRegs<GemvTraits<QT>::REGS>& r) {
  if constexpr (QT == GGML_Q4_K) {
    const uint4 h = load16(blk);                    // d, dmin, scales[12]
    const uint4 a = load16(blk + 16 + q * 32);      // values 0..15 of sub-blocks 2q (low) / 2q+1 (high)
    const uint4 b = load16(blk + 32 + q * 32);      // values 16..31
    r.v[0] = h.x; r.v[1] = h.y; r.v[2] = h.z; r.v[3] = h.w;
    r.v[4] = a.x; r.v[5] = a.y; r.v[6] = a.z; r.v[7] = a.w;
    r.v[8] = b.x; r.v[9] = b.y; r.v[10] = b.z; r.v[11] = b.w;
  } else if constexpr (QT == GGML_Q5_K) {
    const uint4 h = load16(blk);                    // d, dmin, scales[12]
    const uint4 a = load16(blk + 48 + q * 32);      // low nibbles, values 0..15 of sub-blocks 2q / 2q+1
    const uint4 b = load16(blk + 64 + q * 32);      // values 16..31
    const uint4 c = load16(blk + 16), d = load16(blk + 32);   // qh[32]: bit s of qh[l] = bit 4 of sub-block s, lane l
    r.v[0] = h.x; r.v[1] = h.y; r.v[2] = h.z; r.v[3] = h.w;
    r.v[4] = a.x; r.v[5] = a.y; r.v[6] = a.z; r.v[7] = a.w;
    r.v[8] = b.x; r.v[9] = b.y; r.v[10] = b.z; r.v[11] = b.w;
    r.v[12] = c.x; r.v[13] = c.y; r.v[14] = c.z; r.v[15] = c.w;
    r.v[16] = d.x; r.v[17] = d.y; r.v[18] = d.z; r.v[19] = d.w;
  } else if constexpr (QT == GGML_Q6_K) {
    const int h = q >> 1, t = q & 1;
    const uint4 a = load16(blk + 64 * h + 16 * t);          // ql, first 32-byte group of the half
    const uint4 b = load16(blk + 64 * h + 32 + 16 * t);     // ql, second 32-byte group
    const uint4 c = load16(blk + 128 + 32 * h + 16 * t);    // qh
    const uint2 s = load8(blk + 192 + 8 * h);               // int8 scales 8h..8h+7
    r.v[0] = a.x; r.v[1] = a.y; r.v[2] = a.z; r.v[3] = a.w;
    r.v[4] = b.x; r.v[5] = b.y; r.v[6] = b.z; r.v[7] = b.w;
    r.v[8] = c.x; r.v[9] = c.y; r.v[10] = c.z; r.v[11] = c.w;
    r.v[12] = s.x; r.v[13] = s.y;
    r.v[14] = load2(blk + 208);                             // d
  } else {
    const uint8_t* p = blk + q * 68;                        // two 34-byte blocks, 4-byte aligned
    const uint4 a = load16(p), b = load16(p + 16), c = load16(p + 32), d = load16(p + 48);
    r.v[0] = a.x; r.v[1] = a.y; r.v[2] = a.z; r.v[3] = a.w;
    r.v[4] = b.x; r.v[5] = b.y; r.v[6] = b.z; r.v[7] = b.w;
    r.v[8] = c.x; r.v[9] = c.y; r.v[10] = c.z; r.v[11] = c.w;
    r.v[12] = d.x; r.v[13] = d.y; r.v[14] = d.z; r.v[15] = d.w;
    r.v[16] = load4(p + 64);
  }
}

// LDS image of one chunk of quantized activations.
struct ActTile {
  const uint8_t* q8;    // [B][chunk_elems] int8
  const float* xd;      // [B][chunk_sb]  float(half(d)) per 32 values
  const float* xs;      // [B][chunk_sb]  Q4_K: xd * sum(q8) per 32 values
  const int* s16;       // [B][chunk_sb*2] Q6_K: sum(q8) per 16 values
  int chunk_elems;
  int chunk_sb;
};

// Integer sub-block dots of one lane's share of a block.  `dots` receives, for
// Q4_K and Q8_0, the two 32-wide dots of sub-blocks 2q and 2q+1; for Q6_K the
// four 16-wide dots (already minus 32*qsum16) of groups 4h..4h+3, half t.
// The production accumulate below and the block-dot verification export both
// call this function.
template <int QT>
__device__ __forceinline__ void gemv_block_dots(const WeightRegs<GemvTraits<QT>::REGS>& r, int q,
                                                const uint8_t* q8_blk, const int* s16_blk, int (&dots)[4]) {
  if constexpr (QT == GGML_Q4_K) {
    const uint4* xp = reinterpret_cast<const uint4*>(q8_blk + q * 64);
    const uint4 a0 = xp[0], a1 = xp[1], b0 = xp[2], b1 = xp[3];
    int da = 0, db = 0;
    da = dot4(q4k_low(r.v[4]), a0.x, da);  db = dot4(q4k_high(r.v[4]), b0.x, db);
    da = dot4(q4k_low(r.v[5]), a0.y, da);  db = dot4(q4k_high(r.v[5]), b0.y, db);
    da = dot4(q4k_low(r.v[6]), a0.z, da);  db = dot4(q4k_high(r.v[6]), b0.z, db);
    da = dot4(q4k_low(r.v[7]), a0.w, da);  db = dot4(q4k_high(r.v[7]), b0.w, db);
    da = dot4(q4k_low(r.v[8]), a1.x, da);  db = dot4(q4k_high(r.v[8]), b1.x, db);
    da = dot4(q4k_low(r.v[9]), a1.y, da);  db = dot4(q4k_high(r.v[9]), b1.y, db);
    da = dot4(q4k_low(r.v[10]), a1.z, da); db = dot4(q4k_high(r.v[10]), b1.z, db);
    da = dot4(q4k_low(r.v[11]), a1.w, da); db = dot4(q4k_high(r.v[11]), b1.w, db);
    dots[0] = da; dots[1] = db; dots[2] = 0; dots[3] = 0;
  } else if constexpr (QT == GGML_Q5_K) {
    const uint4* xp = reinterpret_cast<const uint4*>(q8_blk + q * 64);
    const uint4 a0 = xp[0], a1 = xp[1], b0 = xp[2], b1 = xp[3];
    const uint32_t xa[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
    const uint32_t xb[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
    int da = 0, db = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t qh = r.v[12 + i] >> (2 * q);               // bit 0: sub-block 2q, bit 1: sub-block 2q+1
      da = dot4(q4k_low(r.v[4 + i]) | ((qh & 0x01010101u) << 4), xa[i], da);
      db = dot4(q4k_high(r.v[4 + i]) | (((qh >> 1) & 0x01010101u) << 4), xb[i], db);
    }
    dots[0] = da; dots[1] = db; dots[2] = 0; dots[3] = 0;
  } else if constexpr (QT == GGML_Q6_K) {
    const int h = q >> 1, t = q & 1;
    const uint8_t* base = q8_blk + h * 128 + t * 16;
    const uint4 x0 = *reinterpret_cast<const uint4*>(base);
    const uint4 x1 = *reinterpret_cast<const uint4*>(base + 32);
    const uint4 x2 = *reinterpret_cast<const uint4*>(base + 64);
    const uint4 x3 = *reinterpret_cast<const uint4*>(base + 96);
    const Q6KQuad u0 = q6k_unpack(r.v[0], r.v[4], r.v[8]);
    const Q6KQuad u1 = q6k_unpack(r.v[1], r.v[5], r.v[9]);
    const Q6KQuad u2 = q6k_unpack(r.v[2], r.v[6], r.v[10]);
    const Q6KQuad u3 = q6k_unpack(r.v[3], r.v[7], r.v[11]);
    int d0 = 0, d1 = 0, d2 = 0, d3 = 0;
    d0 = dot4(u0.g0, x0.x, d0); d1 = dot4(u0.g1, x1.x, d1); d2 = dot4(u0.g2, x2.x, d2); d3 = dot4(u0.g3, x3.x, d3);
    d0 = dot4(u1.g0, x0.y, d0); d1 = dot4(u1.g1, x1.y, d1); d2 = dot4(u1.g2, x2.y, d2); d3 = dot4(u1.g3, x3.y, d3);
    d0 = dot4(u2.g0, x0.z, d0); d1 = dot4(u2.g1, x1.z, d1); d2 = dot4(u2.g2, x2.z, d2); d3 = dot4(u2.g3, x3.z, d3);
    d0 = dot4(u3.g0, x0.w, d0); d1 = dot4(u3.g1, x1.w, d1); d2 = dot4(u3.g2, x2.w, d2); d3 = dot4(u3.g3, x3.w, d3);
    const int* sp = s16_blk + (4 * h) * 2 + t;      // qsum16 of group 4h+j, half t at sp[2j]
    dots[0] = d0 - 32 * sp[0];
    dots[1] = d1 - 32 * sp[2];
    dots[2] = d2 - 32 * sp[4];
    dots[3] = d3 - 32 * sp[6];
  } else {
    const uint4* xp = reinterpret_cast<const uint4*>(q8_blk + q * 64);
    const uint4 a0 = xp[0], a1 = xp[1], b0 = xp[2], b1 = xp[3];
    int da = 0, db = 0;
    // first block: quants start 2 bytes into the registers
    da = dot4(__builtin_amdgcn_alignbit(r.v[1], r.v[0], 16), a0.x, da);
    da = dot4(__builtin_amdgcn_alignbit(r.v[2], r.v[1], 16), a0.y, da);
    da = dot4(__builtin_amdgcn_alignbit(r.v[3], r.v[2], 16), a0.z, da);
    da = dot4(__builtin_amdgcn_alignbit(r.v[4], r.v[3], 16), a0.w, da);
    da = dot4(__builtin_amdgcn_alignbit(r.v[5], r.v[4], 16), a1.x, da);
    da = dot4(__builtin_amdgcn_alignbit(r.v[6], r.v[5], 16), a1.y, da);
    da = dot4(__builtin_amdgcn_alignbit(r.v[7], r.v[6], 16), a1.z, da);
    da = dot4(__builtin_amdgcn_alignbit(r.v[8], r.v[7], 16), a1.w, da);
    // second block: header in the top half of v[8], quants dword aligned from v[9]
    db = dot4(r.v[9], b0.x, db);  db = dot4(r.v[10], b0.y, db);
    db = dot4(r.v[11], b0.z, db); db = dot4(r.v[12], b0.w, db);
    db = dot4(r.v[13], b1.x, db); db = dot4(r.v[14], b1.y, db);
    db = dot4(r.v[15], b1.z, db); db = dot4(r.v[16], b1.w, db);
    dots[0] = da; dots[1] = db; dots[2] = 0; dots[3] = 0;
  }
}

// Per-lane float32 factors of one block that do not depend on the batch row.
template <int QT>
struct BlockScales {
  float f[4];   // multiplies xd*dot      (Q4_K: d*sc; Q6_K: d*sc16; Q8_0: d)
  float m[2];   // Q4_K only: dmin*mn
};

template <int QT>
__device__ __forceinline__ BlockScales<QT> gemv_block_scales(const WeightRegs<GemvTraits<QT>::REGS>& r, int q) {
  BlockScales<QT> s;
  if constexpr (gemv_has_mins(QT)) {
    const Q4KScales u = q4k_unpack_scales(r.v[1], r.v[2], r.v[3]);
    const float d = f16_bits_to_float(r.v[0] & 0xFFFFu), dmin = f16_bits_to_float(r.v[0] >> 16);
    // sub-blocks 2q and 2q+1 sit in bytes 2(q&1), 2(q&1)+1 of the low (q<2) or high word
    const uint32_t scw = ((q & 2) ? u.sc_hi : u.sc_lo) >> (16 * (q & 1));
    const uint32_t mnw = ((q & 2) ? u.mn_hi : u.mn_lo) >> (16 * (q & 1));
    s.f[0] = d * static_cast<float>(scw & 0xFFu);
    s.f[1] = d * static_cast<float>((scw >> 8) & 0xFFu);
    s.f[2] = 0.0f; s.f[3] = 0.0f;
    s.m[0] = dmin * static_cast<float>(mnw & 0xFFu);
    s.m[1] = dmin * static_cast<float>((mnw >> 8) & 0xFFu);
  } else if constexpr (QT == GGML_Q6_K) {
    const int t = q & 1;
    const float d = f16_bits_to_float(r.v[14]);
    const uint32_t lo = r.v[12] >> (8 * t), hi = r.v[13] >> (8 * t);   // byte 0: index t, byte 2: index 2+t
    s.f[0] = d * static_cast<float>(static_cast<int8_t>(lo & 0xFFu));
    s.f[1] = d * static_cast<float>(static_cast<int8_t>((lo >> 16) & 0xFFu));
    s.f[2] = d * static_cast<float>(static_cast<int8_t>(hi & 0xFFu));
    s.f[3] = d * static_cast<float>(static_cast<int8_t>((hi >> 16) & 0xFFu));
    s.m[0] = 0.0f; s.m[1] = 0.0f;
  } else {
    s.f[0] = f16_bits_to_float(r.v[0] & 0xFFFFu);
    s.f[1] = f16_bits_to_float(r.v[8] >> 16);
    s.f[2] = 0.0f; s.f[3] = 0.0f;
    s.m[0] = 0.0f; s.m[1] = 0.0f;
  }
  return s;
}

// One lane's contribution of one block to one batch row.
template <int QT>
__device__ __forceinline__ float gemv_block_term(const WeightRegs<GemvTraits<QT>::REGS>& r, const BlockScales<QT>& s,
                                                 int q, const ActTile& t, int b, int blk_local) {
  const uint8_t* q8_blk = t.q8 + b * t.chunk_elems + blk_local * QK_K;
  const int sb0 = b * t.chunk_sb + blk_local * 8;
  int dots[4];
  gemv_block_dots<QT>(r, q, q8_blk, QT == GGML_Q6_K ? t.s16 + sb0 * 2 : nullptr, dots);
  if constexpr (gemv_has_mins(QT)) {
    const float2 xd = *reinterpret_cast<const float2*>(t.xd + sb0 + 2 * q);
    const float2 xs = *reinterpret_cast<const float2*>(t.xs + sb0 + 2 * q);
    float v = s.f[0] * (xd.x * static_cast<float>(dots[0]));
    v += s.f[1] * (xd.y * static_cast<float>(dots[1]));
    v -= s.m[0] * xs.x;
    v -= s.m[1] * xs.y;
    return v;
  } else if constexpr (QT == GGML_Q6_K) {
    const float4 xd = *reinterpret_cast<const float4*>(t.xd + sb0 + 4 * (q >> 1));
    float v = s.f[0] * (xd.x * static_cast<float>(dots[0]));
    v += s.f[1] * (xd.y * static_cast<float>(dots[1]));
    v += s.f[2] * (xd.z * static_cast<float>(dots[2]));
    v += s.f[3] * (xd.w * static_cast<float>(dots[3]));
    return v;
  } else {
    const float2 xd = *reinterpret_cast<const float2*>(t.xd + sb0 + 2 * q);
    float v = s.f[0] * (xd.x * static_cast<float>(dots[0]));
    v += s.f[1] * (xd.y * static_cast<float>(dots[1]));
    return v;
  }
}

// Quantize (or, for KIND_Q8_1 input, unpack) the activations of K-blocks
// [kc, kc + chunk_blocks) of `rows` batch rows into LDS.  Eight lanes share a
// 32-value group.  q8_1 GEMV convention: d = amax/127 (float32), q =
// clamp(roundf(x/d), -128, 127), consumers see float(half(d))
// (gguf_q4_k_gemv.hip:740-772).  Rows >= rows are zero filled.
template <int QT, int B>
__device__ __forceinline__ void gemv_stage_activations(const GemvArgs& a, int kc, int chunk_blocks, uint8_t* q8,
                                                       float* xd_out, float* xs_out, int* s16_out, int chunk_elems,
                                                       int chunk_sb) {
  const int tid = threadIdx.x;
  const int team = tid >> 3, e = tid & 7, nteams = blockDim.x >> 3;
  const int nb = a.K / QK_K;
  const int blocks_here = min(chunk_blocks, nb - kc);
  const int groups = blocks_here * 8;
  // (batch row, group) pairs over all the teams at once: with few groups per row (a short K chunk and many rows)
  // a loop over the rows outside would leave most teams idle and make the rows' loads a chain of round trips
  {
    for (int idx = team; idx < B * groups; idx += nteams) {
      const int b = B == 1 ? 0 : idx / groups;
      const int j = B == 1 ? idx : idx - b * groups;
      uint32_t packed = 0;
      float xd = 0.0f;
      if (b < a.rows) {
        if (a.x_kind == KIND_Q8_1) {
          const uint8_t* blk = static_cast<const uint8_t*>(a.x) +
                               (static_cast<int64_t>(b) * (a.K / 32) + kc * 8 + j) * Q8_1_BYTES;
          packed = *reinterpret_cast<const uint32_t*>(blk + 4 + 4 * e);
          xd = f16_bits_to_float(*reinterpret_cast<const uint32_t*>(blk) & 0xFFFFu);
        } else {
          const int64_t k0 = static_cast<int64_t>(b) * a.K + kc * QK_K + j * 32 + e * 4;
          float v0, v1, v2, v3;
          if (a.x_kind == KIND_F32) {
            const float4 v = *reinterpret_cast<const float4*>(static_cast<const float*>(a.x) + k0);
            v0 = v.x; v1 = v.y; v2 = v.z; v3 = v.w;
          } else {
            const uint2 v = *reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(a.x) + k0);
            if (a.x_kind == KIND_BF16 || a.x_kind == KIND_SILU_BF16) {
              v0 = bf16_bits_to_float(v.x & 0xFFFFu); v1 = bf16_bits_to_float(v.x >> 16);
              v2 = bf16_bits_to_float(v.y & 0xFFFFu); v3 = bf16_bits_to_float(v.y >> 16);
              if (a.x_kind == KIND_SILU_BF16) {
                const uint2 u = *reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(a.x_up) + k0);
                const auto act = [](float g, uint32_t up_bits) {
                  const float silu = g / (1.0f + expf(-g));
                  return bf16_bits_to_float(float_to_bf16_bits(silu * bf16_bits_to_float(up_bits)));
                };
                v0 = act(v0, u.x & 0xFFFFu); v1 = act(v1, u.x >> 16);
                v2 = act(v2, u.y & 0xFFFFu); v3 = act(v3, u.y >> 16);
              }
            } else {
              v0 = f16_bits_to_float(v.x & 0xFFFFu); v1 = f16_bits_to_float(v.x >> 16);
              v2 = f16_bits_to_float(v.y & 0xFFFFu); v3 = f16_bits_to_float(v.y >> 16);
            }
          }
          const float amax = oct_max(fmaxf(fmaxf(fabsf(v0), fabsf(v1)), fmaxf(fabsf(v2), fabsf(v3))));
          const float d = amax / 127.0f;
          if (amax != 0.0f) {
            const int q0 = max(-128, min(127, static_cast<int>(roundf(v0 / d))));
            const int q1 = max(-128, min(127, static_cast<int>(roundf(v1 / d))));
            const int q2 = max(-128, min(127, static_cast<int>(roundf(v2 / d))));
            const int q3 = max(-128, min(127, static_cast<int>(roundf(v3 / d))));
            packed = (q0 & 0xFF) | ((q1 & 0xFF) << 8) | ((q2 & 0xFF) << 16) | (static_cast<uint32_t>(q3 & 0xFF) << 24);
          }
          xd = static_cast<float>(static_cast<half_t>(d));
        }
      }
      *reinterpret_cast<uint32_t*>(q8 + b * chunk_elems + j * 32 + e * 4) = packed;
      const int part = dot4(0x01010101u, packed, 0);
      if constexpr (QT == GGML_Q6_K) {
        int h = part;
        h += dpp_i<DPP_QUAD_XOR1>(h);
        h += dpp_i<DPP_QUAD_XOR2>(h);
        if ((e & 3) == 0) s16_out[(b * chunk_sb + j) * 2 + (e >> 2)] = h;
        if (e == 0) xd_out[b * chunk_sb + j] = xd;
      } else {
        const int total = oct_sum_i(part);
        if (e == 0) {
          xd_out[b * chunk_sb + j] = xd;
          if constexpr (gemv_has_mins(QT)) xs_out[b * chunk_sb + j] = xd * static_cast<float>(total);
        }
      }
    }
  }
}

// Bytes of dynamic LDS the kernel needs.
inline size_t gemv_lds_bytes(int qt, int B, int R, int CB, int ks, int nrg) {
  const size_t chunk_elems = static_cast<size_t>(ks) * CB * QK_K;
  const size_t chunk_sb = chunk_elems / 32;
  size_t bytes = B * chunk_elems;                       // q8
  bytes += B * chunk_sb * 4;                            // xd
  if (gemv_has_mins(qt)) bytes += B * chunk_sb * 4;     // xs
  if (qt == GGML_Q6_K) bytes += B * chunk_sb * 8;       // s16
  bytes += static_cast<size_t>(ks) * nrg * 16 * R * B * 4;  // K-slice reduction
  return bytes;
}

// `w_row0` / `out` already point at the matrix this workgroup column works on;
// `first_row` is the first output row of the workgroup.
// `emit(b, row, value)` receives each finished output once (batch row b, output
// row `row` < N), from the thread that summed its K-slices.  A caller that runs
// the body more than once in a kernel separates the calls with a barrier, as
// the LDS staging area is reused.
//
// DUAL (R == 2, B == 1): the lane's two rows are the SAME row index of two matrices
// `w` and `w2` (a gate/up pair), so one pass with one staging of the activations
// yields both; the workgroup then owns nrg*16 output rows and `emit` receives the
// matrix (0 or 1) in place of the batch row.
template <int QT, int B, int R, int CB, bool DUAL = false, class Emit>
__device__ __forceinline__ void gemv_workgroup_emit(const GemvArgs& a, const uint8_t* w, int first_row, uint8_t* smem,
                                                    Emit emit, const uint8_t* w2 = nullptr) {
  static_assert(!DUAL || (R == 2 && B == 1), "the dual form pairs two matrices at batch 1");
  using Regs = WeightRegs<GemvTraits<QT>::REGS>;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int kslice = wave % a.ks, rowgrp = wave / a.ks;
  const int q = lane & 3, rg = lane >> 2;
  const int rows_wg = a.nrg * 16 * R;
  const int nb = a.K / QK_K;
  const int chunk_blocks = a.ks * CB;
  const int chunk_elems = chunk_blocks * QK_K, chunk_sb = chunk_blocks * 8;
  const int64_t row_bytes = static_cast<int64_t>(nb) * GemvTraits<QT>::SUPER_BYTES;

  uint8_t* q8 = smem;
  float* xd = reinterpret_cast<float*>(q8 + B * chunk_elems);
  float* xs = xd + B * chunk_sb;
  int* s16 = reinterpret_cast<int*>(xs);
  float* red = gemv_has_mins(QT) ? xs + B * chunk_sb
             : (QT == GGML_Q6_K) ? reinterpret_cast<float*>(s16 + B * chunk_sb * 2)
                                 : xs;

  const uint8_t* wrow[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int row = DUAL ? min(first_row + rowgrp * 16 + rg, a.N - 1)
                         : min(first_row + rowgrp * 16 * R + 16 * r + rg, a.N - 1);
    wrow[r] = ((DUAL && r == 1) ? w2 : w) + static_cast<int64_t>(row) * row_bytes;
  }

  float acc[R][B];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int b = 0; b < B; ++b) acc[r][b] = 0.0f;

  ActTile tile{q8, xd, xs, s16, chunk_elems, chunk_sb};

  for (int kc = 0; kc < nb; kc += chunk_blocks) {
    Regs wr[R][CB];
#pragma unroll
    for (int c = 0; c < CB; ++c) {
      const int kb = kc + kslice * CB + c;
      if (kb < nb) {
#pragma unroll
        for (int r = 0; r < R; ++r)
          gemv_load_block<QT>(wrow[r] + static_cast<int64_t>(kb) * GemvTraits<QT>::SUPER_BYTES, q, wr[r][c]);
      }
    }
    if (kc > 0) __syncthreads();   // every wave is done reading the previous chunk
    gemv_stage_activations<QT, B>(a, kc, chunk_blocks, q8, xd, xs, s16, chunk_elems, chunk_sb);
    __syncthreads();
#pragma unroll
    for (int c = 0; c < CB; ++c) {
      const int kb = kc + kslice * CB + c;
      if (kb < nb) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const BlockScales<QT> s = gemv_block_scales<QT>(wr[r][c], q);
#pragma unroll
          for (int b = 0; b < B; ++b) acc[r][b] += gemv_block_term<QT>(wr[r][c], s, q, tile, b, kslice * CB + c);
        }
      }
    }
  }

  // quad reduce, then K-slice reduce through LDS
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int b = 0; b < B; ++b) {
      const float v = quad_sum(acc[r][b]);
      if (q == 0) red[(kslice * B + b) * rows_wg + rowgrp * 16 * R + 16 * r + rg] = v;
    }
  __syncthreads();
  for (int idx = tid; idx < rows_wg * B; idx += blockDim.x) {
    const int b = idx / rows_wg, rl = idx - b * rows_wg;
    const int which = (rl >> 4) & 1;                                  // DUAL: 16 rows of w, then 16 of w2, per row group
    const int row = DUAL ? first_row + (rl >> 5) * 16 + (rl & 15) : first_row + rl;
    if (row < a.N && b < a.rows) {
      float v = 0.0f;
      for (int s = 0; s < a.ks; ++s) v += red[(s * B + b) * rows_wg + rl];
      emit(DUAL ? which : b, row, v);
    }
  }
}

template <int QT, int B, int R, int CB>
__device__ __forceinline__ void gemv_workgroup(const GemvArgs& a, const uint8_t* w, int first_row, uint8_t* smem) {
  gemv_workgroup_emit<QT, B, R, CB, false>(a, w, first_row, smem, [&](int b, int row, float v) {
    store_scalar(a.out, static_cast<int64_t>(b) * a.N + row, v, a.out_kind);
  });
}

}  // namespace hipengine_gfx950
