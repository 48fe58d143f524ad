// "Run" form of the q8_1 decode GEMV: every wave owns G whole consecutive rows
// and streams them as ONE contiguous run of G*nb 256-value blocks.
//
// A wave-wide load covers 16 consecutive blocks (4 lanes per block), i.e. 2304
// contiguous bytes of Q4_K: measured on MI355X this reads a 50 MB weight within
// ~10% of a plain coalesced copy, where the row-strided layout of
// gguf_gemv.hpp (16 different rows per load) is ~30% slower.  G is chosen so
// that G*nb is a multiple of 16, which makes the run a whole number m of wave
// loads; lane quad j of load i holds block 16*i + j of the run, which belongs
// to row (16*i + j) / nb and K block (16*i + j) % nb.
//
// Consequences:
//   * no K split and no cross-wave reduction: a row's m*16/G blocks all live in
//     one wave; the only workgroup barrier is the one after activation staging;
//   * activations for the whole K are quantized to q8_1 once per workgroup into
//     LDS (a workgroup is several waves = several runs sharing them);
//   * different lanes of a load need different K blocks, so the LDS image pads
//     every block (272 or 288 bytes apart) to keep the 16-byte reads of a
//     quarter wave on distinct banks;
//   * each lane keeps G accumulators and adds its term to the one its block
//     belongs to; rows are reduced across the wave with DPP at the end.
//
// The integer dots, the scale decode and the float32 combine are the functions
// of gguf_gemv.hpp, so both kernels produce bit-identical sub-block dots.
#pragma once

#include "gguf_gemv.hpp"

namespace hipengine_gfx950 {

struct GemvRunArgs {
  const void* x;
  const uint8_t* w;
  void* out;
  int x_kind;
  int out_kind;
  int rows;     // batch rows, 1..B
  int K;
  int N;
  int waves;    // waves (= runs) per workgroup
};

template <int QT>
constexpr int run_q8_stride() {
  return QT == GGML_Q6_K ? 288 : 272;
}

// Bytes of dynamic LDS: per batch row nb padded q8 blocks, nb*64 bytes of
// scale records and, for Q6_K, nb*64 bytes of 16-wide q8 sums.
inline size_t gemv_run_lds_bytes(int qt, int B, int K) {
  const size_t nb = K / QK_K;
  const size_t stride = qt == GGML_Q6_K ? 288 : 272;
  return B * nb * (stride + 64 + (qt == GGML_Q6_K ? 64 : 0));
}

// amax / 127.0f, correctly rounded, in three operations: q = a*c, r = fma(-q, 127, a),
// q' = fma(r, c, q) with c = RN(1/127).  Equal to the IEEE quotient for every finite
// non-negative float (checked exhaustively on the host over all 2^31 - 2^23 values).
__device__ __forceinline__ float div_by_127(float a) {
  const float c = 1.0f / 127.0f;
  const float q = a * c;
  return __builtin_fmaf(__builtin_fmaf(-q, 127.0f, a), c, q);
}

// One lane's share of a 32-value activation group (4 lanes x 8 values): quantize the
// fetched values to q8_1 (or take them from a q8_1 block) -> 8 packed int8 and the
// group's scale, rounded to half as the q8_1 block stores it.  raw: 8 floats, or 8
// halves/bf16 in raw[0..3], or for q8_1 input the lane's 8 quants in raw[0..1] and the
// block's {d, s} halves in raw[2].
//
// q = clamp(roundf(v / d), -128, 127) goes through the reciprocal: t = v * rcp(d) is within
// 3e-5 of the quotient (|v/d| <= 127, reciprocal good to 1 ulp).  t + 1.5*2^23 rounds t to
// the nearest integer r and leaves r's two's complement in the low mantissa bits; unless t
// is within 1e-4 of a tie, r equals roundf(v/d).  Near ties, and scales in the denormal
// range where the reciprocal overflows, redo the lane's values with the IEEE division.
// Bit-exact with the direct evaluation.
__device__ __forceinline__ void q8_quantize8(int x_kind, const uint32_t (&raw)[8], bool present, uint32_t (&packed)[2],
                                             float& xd) {
  packed[0] = 0; packed[1] = 0;
  xd = 0.0f;
  if (!present) return;
  if (x_kind == KIND_Q8_1) {
    packed[0] = raw[0]; packed[1] = raw[1];
    xd = f16_bits_to_float(raw[2] & 0xFFFFu);
    return;
  }
  float v[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    if (x_kind == KIND_F32) v[i] = bits_to_float(raw[i]);
    else if (x_kind == KIND_BF16) v[i] = bf16_bits_to_float((raw[i >> 1] >> (16 * (i & 1))) & 0xFFFFu);
    else v[i] = f16_bits_to_float((raw[i >> 1] >> (16 * (i & 1))) & 0xFFFFu);
  }
  float m = fmaxf(fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3]))),
                  fmaxf(fmaxf(fabsf(v[4]), fabsf(v[5])), fmaxf(fabsf(v[6]), fabsf(v[7]))));
  uint32_t u = float_to_bits(m);                       // non-negative: integer order = float order
  u = max(u, static_cast<uint32_t>(dpp_i<DPP_QUAD_XOR1>(static_cast<int>(u))));
  u = max(u, static_cast<uint32_t>(dpp_i<DPP_QUAD_XOR2>(static_cast<int>(u))));
  const float amax = bits_to_float(u);
  const float d = div_by_127(amax);
  if (amax != 0.0f) {
    constexpr float MAGIC = 12582912.0f;
    const float inv = __builtin_amdgcn_rcpf(d);
    float mg[8], worst = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float t = v[i] * inv;
      mg[i] = t + MAGIC;
      worst = __builtin_fmaxf(worst, fabsf(t - (mg[i] - MAGIC)));
    }
    packed[0] = __builtin_amdgcn_perm(float_to_bits(mg[1]), float_to_bits(mg[0]), 0x0c0c0400u) |
                __builtin_amdgcn_perm(float_to_bits(mg[3]), float_to_bits(mg[2]), 0x04000c0cu);
    packed[1] = __builtin_amdgcn_perm(float_to_bits(mg[5]), float_to_bits(mg[4]), 0x0c0c0400u) |
                __builtin_amdgcn_perm(float_to_bits(mg[7]), float_to_bits(mg[6]), 0x04000c0cu);
    if (__builtin_expect(worst > 0.4999f || d < 1.0e-30f, 0)) {
      uint32_t p[2] = {0u, 0u};
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int q = max(-128, min(127, static_cast<int>(roundf(v[i] / d))));
        p[i >> 2] |= static_cast<uint32_t>(q & 0xFF) << (8 * (i & 3));
      }
      packed[0] = p[0]; packed[1] = p[1];
    }
  }
  xd = static_cast<float>(static_cast<half_t>(d));
}

// Whole-K activation staging for the run and stream kernels: teams of 4 lanes take one
// 32-value group each, 8 values per lane.
//   q8   : [B][nb] blocks, Q8S bytes apart
//   rec  : [B][nb][4] 16-byte records, one per lane q of a block:
//            Q4_K {xd(2q), xd(2q+1), xd*qsum(2q), xd*qsum(2q+1)}
//            Q8_0 {xd(2q), xd(2q+1), -, -}
//            Q6_K {xd(4h), xd(4h+1), xd(4h+2), xd(4h+3)}, q = 2h+t
//   s16  : Q6_K only, [B][nb][4] x {qsum16(4h+j, half t)} j = 0..3
//
// Split in two so that a kernel can put the activation loads in front of its weight
// loads: vmcnt counts loads in issue order, so waiting for activations issued AFTER
// the weight ring would also wait for the ring.
//   stage_fetch  : issue the loads of this thread's first S groups per batch row
//   stage_commit : quantize them into LDS; groups beyond the first S per thread
//                  are loaded and quantized here (large K only)
template <int B, int S>
struct StageRegs {
  uint32_t raw[B][S][8];
};

// The lane's 8 values of group j of one batch row (or its share of a q8_1 block).
__device__ __forceinline__ void gemv_run_fetch8(const GemvRunArgs& a, int b, int j, int e, uint32_t (&raw)[8]) {
#pragma unroll
  for (int i = 0; i < 8; ++i) raw[i] = 0u;
  if (a.x_kind == KIND_F32) {
    const uint4* src = reinterpret_cast<const uint4*>(static_cast<const float*>(a.x) + static_cast<int64_t>(b) * a.K + j * 32 + e * 8);
    const uint4 lo = src[0], hi = src[1];
    raw[0] = lo.x; raw[1] = lo.y; raw[2] = lo.z; raw[3] = lo.w;
    raw[4] = hi.x; raw[5] = hi.y; raw[6] = hi.z; raw[7] = hi.w;
  } else if (a.x_kind == KIND_Q8_1) {
    const uint8_t* blk = static_cast<const uint8_t*>(a.x) + (static_cast<int64_t>(b) * (a.K / 32) + j) * Q8_1_BYTES;
    raw[0] = *reinterpret_cast<const uint32_t*>(blk + 4 + 8 * e);
    raw[1] = *reinterpret_cast<const uint32_t*>(blk + 8 + 8 * e);
    raw[2] = *reinterpret_cast<const uint32_t*>(blk);
  } else {
    const uint4 h = *reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(a.x) + static_cast<int64_t>(b) * a.K + j * 32 + e * 8);
    raw[0] = h.x; raw[1] = h.y; raw[2] = h.z; raw[3] = h.w;
  }
}

template <int QT, int B, int S>
__device__ __forceinline__ void gemv_run_stage_fetch(const GemvRunArgs& a, StageRegs<B, S>& sr) {
  const int tid = threadIdx.x;
  const int team = tid >> 2, e = tid & 3, nteams = blockDim.x >> 2;
  const int groups = (a.K / QK_K) * 8;
#pragma unroll
  for (int b = 0; b < B; ++b) {
#pragma unroll
    for (int s = 0; s < S; ++s) {
      const int j = team + s * nteams;
      if (b < a.rows && j < groups) {
        gemv_run_fetch8(a, b, j, e, sr.raw[b][s]);
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) sr.raw[b][s][i] = 0u;
      }
    }
  }
}

// Quantize one fetched group (8 values of one lane) and write it to the LDS image.
template <int QT>
__device__ __forceinline__ void gemv_run_stage_one(int x_kind, const uint32_t (&raw)[8], bool present, int j, int e,
                                                   uint8_t* q8_row, float* rec_row, int* s16_row) {
  constexpr int Q8S = run_q8_stride<QT>();
  uint32_t packed[2];
  float xd;
  q8_quantize8(x_kind, raw, present, packed, xd);
  const int kb = j >> 3, sb = j & 7;
  *reinterpret_cast<uint2*>(q8_row + kb * Q8S + sb * 32 + e * 8) = make_uint2(packed[0], packed[1]);
  const int part = dot4(0x01010101u, packed[1], dot4(0x01010101u, packed[0], 0));
  float* r = rec_row + kb * 16;
  if constexpr (QT == GGML_Q6_K) {
    const int h16 = part + dpp_i<DPP_QUAD_XOR1>(part);   // lanes 0,1: values 0..15; lanes 2,3: values 16..31
    // group sb = 4h + jj, half t = e>>1 -> record of lane q = 2h+t, slot jj
    const int h = sb >> 2, jj = sb & 3;
    if ((e & 1) == 0) s16_row[kb * 16 + (2 * h + (e >> 1)) * 4 + jj] = h16;
    if (e == 0) {   // xd of group sb goes to both records (t = 0, 1) of half h
      r[(2 * h) * 4 + jj] = xd;
      r[(2 * h + 1) * 4 + jj] = xd;
    }
  } else {
    int total = part + dpp_i<DPP_QUAD_XOR1>(part);
    total += dpp_i<DPP_QUAD_XOR2>(total);
    if (e == 0) {   // sub-block sb -> record of lane q = sb>>1, slot sb&1 (+2 for the xd*qsum term)
      r[(sb >> 1) * 4 + (sb & 1)] = xd;
      if constexpr (gemv_has_mins(QT)) r[(sb >> 1) * 4 + 2 + (sb & 1)] = xd * static_cast<float>(total);
    }
  }
}

// ALL_UP_FRONT: the caller guarantees that the S groups per thread fetched up front cover the row
// (K/32 <= S * threads/4); the loop over the rest is then not generated.
template <int QT, int B, int S, bool ALL_UP_FRONT = false>
__device__ __forceinline__ void gemv_run_stage_commit(const GemvRunArgs& a, const StageRegs<B, S>& sr, uint8_t* q8,
                                                      float* rec, int* s16) {
  constexpr int Q8S = run_q8_stride<QT>();
  const int tid = threadIdx.x;
  const int team = tid >> 2, e = tid & 3, nteams = blockDim.x >> 2;
  const int nb = a.K / QK_K;
  const int groups = nb * 8;
#pragma unroll
  for (int b = 0; b < B; ++b) {
    uint8_t* q8_row = q8 + b * nb * Q8S;
    float* rec_row = rec + b * nb * 16;
    int* s16_row = s16 + b * nb * 16;
#pragma unroll
    for (int s = 0; s < S; ++s) {
      const int j = team + s * nteams;
      if (j < groups) gemv_run_stage_one<QT>(a.x_kind, sr.raw[b][s], b < a.rows, j, e, q8_row, rec_row, s16_row);
    }
  }
  // large K or batch: the rest - (batch row, group) items past the first S groups per row - is loaded here, P
  // items per thread at a time across the batch rows, so that a load latency is paid once per P items
  // and not once per item per row
  const int rest = ALL_UP_FRONT ? 0 : groups - S * nteams;   // groups per row still to do (may be <= 0)
  if (rest > 0) {
    constexpr int P = B >= 4 ? 8 : 2;
    const int per_row = (rest + nteams - 1) / nteams;  // items of this team per batch row
    const int items = per_row * B;
    int b0 = 0, r0 = 0;                               // batch row and per-row index of item i0 (no division)
    for (int i0 = 0; i0 < items; i0 += P) {
      uint32_t raw[P][8];
      int b = b0, r = r0;
#pragma unroll
      for (int p = 0; p < P; ++p) {
        const int j = team + (S + r) * nteams;
        if (b < a.rows && j < groups) {               // b >= B only past the last item; then b >= a.rows too
          gemv_run_fetch8(a, b, j, e, raw[p]);
        } else {
#pragma unroll
          for (int i = 0; i < 8; ++i) raw[p][i] = 0u;
        }
        if (++r == per_row) { r = 0; ++b; }
      }
      b = b0; r = r0;
#pragma unroll
      for (int p = 0; p < P; ++p) {
        const int j = team + (S + r) * nteams;
        if (b < B && j < groups)
          gemv_run_stage_one<QT>(a.x_kind, raw[p], b < a.rows, j, e, q8 + b * nb * Q8S, rec + b * nb * 16, s16 + b * nb * 16);
        if (++r == per_row) { r = 0; ++b; }
      }
      b0 = b; r0 = r;
    }
  }
}

// One lane's float32 contribution of one block to one batch row, run layout.
template <int QT>
__device__ __forceinline__ float gemv_run_block_term(const WeightRegs<GemvTraits<QT>::REGS>& r, const BlockScales<QT>& s,
                                                     int q, const uint8_t* q8_blk, const float* rec_blk,
                                                     const int* s16_blk) {
  int dots[4];
  if constexpr (QT == GGML_Q6_K) {
    // gemv_block_dots expects the qsum16 of group g, half t at s16[g*2 + t]; the run
    // records keep the four a lane needs together, so subtract them here instead.
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
    const int4 sq = *reinterpret_cast<const int4*>(s16_blk + q * 4);
    dots[0] = d0 - 32 * sq.x; dots[1] = d1 - 32 * sq.y; dots[2] = d2 - 32 * sq.z; dots[3] = d3 - 32 * sq.w;
    const float4 xd = *reinterpret_cast<const float4*>(rec_blk + q * 4);
    float v = s.f[0] * (xd.x * static_cast<float>(dots[0]));
    v += s.f[1] * (xd.y * static_cast<float>(dots[1]));
    v += s.f[2] * (xd.z * static_cast<float>(dots[2]));
    v += s.f[3] * (xd.w * static_cast<float>(dots[3]));
    return v;
  } else {
    gemv_block_dots<QT>(r, q, q8_blk, nullptr, dots);
    const float4 rc = *reinterpret_cast<const float4*>(rec_blk + q * 4);
    float v = s.f[0] * (rc.x * static_cast<float>(dots[0]));
    v += s.f[1] * (rc.y * static_cast<float>(dots[1]));
    if constexpr (gemv_has_mins(QT)) {
      v -= s.m[0] * rc.z;
      v -= s.m[1] * rc.w;
    }
    return v;
  }
}

constexpr int DPP_ROW_MIRROR = 0x140;
constexpr int DPP_ROW_BCAST15 = 0x142;
constexpr int DPP_ROW_BCAST31 = 0x143;

// Sum over the 64 lanes of a wave; the total is valid in lane 63.
__device__ __forceinline__ float wave_sum_to_lane63(float v) {
  v += dpp_f<DPP_QUAD_XOR1>(v);
  v += dpp_f<DPP_QUAD_XOR2>(v);
  v += dpp_f<DPP_ROW_HALF_MIRROR>(v);
  v += dpp_f<DPP_ROW_MIRROR>(v);     // every lane of a row of 16 now holds the row total
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), DPP_ROW_BCAST15, 0xA, 0xF, false));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), DPP_ROW_BCAST31, 0xC, 0xF, false));
  return v;
}

// ALL_UP_FRONT: the two activation groups per thread fetched up front cover K (K/32 <= 2 * threads/4).
template <int QT, int B, int G, int CB, bool ALL_UP_FRONT = false>
__device__ __forceinline__ void gemv_run_workgroup(const GemvRunArgs& a, uint8_t* smem) {
  using Regs = WeightRegs<GemvTraits<QT>::REGS>;
  constexpr int Q8S = run_q8_stride<QT>();
  constexpr int SUPER = GemvTraits<QT>::SUPER_BYTES;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int q = lane & 3, j = lane >> 2;
  const int nb = a.K / QK_K;
  const int m = G * nb / 16;                                  // wave loads per run
  const int64_t run = static_cast<int64_t>(blockIdx.x) * a.waves + wave;
  const int64_t first_row = run * G;
  const int64_t total_blocks = static_cast<int64_t>(a.N) * nb;
  const int64_t run_block0 = first_row * nb;

  uint8_t* q8 = smem;
  float* rec = reinterpret_cast<float*>(q8 + B * nb * Q8S);
  int* s16 = reinterpret_cast<int*>(rec + B * nb * 16);

  float acc[G][B];
#pragma unroll
  for (int g = 0; g < G; ++g)
#pragma unroll
    for (int b = 0; b < B; ++b) acc[g][b] = 0.0f;

  // position of this lane's block inside the run: K block kb and row r of load i
  int kb = j % nb, r = j / nb;
  const int step_r = 16 / nb, step_kb = 16 % nb;   // advance of (r, kb) per load

  // activation loads first, then the weight loads, then the quantization: the wait
  // for the activations must not include the (later issued) weight loads
  constexpr int S = 2;
  StageRegs<B, S> sr;
  gemv_run_stage_fetch<QT, B, S>(a, sr);

  for (int i0 = 0; i0 < m; i0 += CB) {
    Regs wr[CB];
#pragma unroll
    for (int c = 0; c < CB; ++c) {
      if (i0 + c < m) {
        int64_t blk = run_block0 + static_cast<int64_t>(i0 + c) * 16 + j;
        blk = blk < total_blocks ? blk : total_blocks - 1;   // runs past the last row re-read its last block
        gemv_load_block<QT>(a.w + blk * SUPER, q, wr[c]);
      }
    }
    if (i0 == 0) {
      gemv_run_stage_commit<QT, B, S, ALL_UP_FRONT>(a, sr, q8, rec, s16);
      __syncthreads();
    }
#pragma unroll
    for (int c = 0; c < CB; ++c) {
      if (i0 + c < m) {
        const BlockScales<QT> s = gemv_block_scales<QT>(wr[c], q);
#pragma unroll
        for (int b = 0; b < B; ++b) {
          const float term = gemv_run_block_term<QT>(wr[c], s, q, q8 + (b * nb + kb) * Q8S, rec + (b * nb + kb) * 16,
                                                     s16 + (b * nb + kb) * 16);
#pragma unroll
          for (int g = 0; g < G; ++g) acc[g][b] += (r == g) ? term : 0.0f;
        }
        kb += step_kb;
        r += step_r;
        if (kb >= nb) { kb -= nb; r += 1; }
      }
    }
  }

#pragma unroll
  for (int g = 0; g < G; ++g)
#pragma unroll
    for (int b = 0; b < B; ++b) {
      const float v = wave_sum_to_lane63(acc[g][b]);
      const int64_t row = first_row + g;
      if (lane == 63 && row < a.N && b < a.rows) store_scalar(a.out, static_cast<int64_t>(b) * a.N + row, v, a.out_kind);
    }
}

}  // namespace hipengine_gfx950
