// "Tile" form of the q8_1 decode GEMV for Q4_K weights, batch 1..8, on the int8
// MFMA: every byte of the weight is requested from HBM in the first
// microsecond of the kernel, and the dots run on the matrix pipe.
//
// Why: at decode sizes (50 MB of weights = 6 us of HBM time) the kernel is
// bound by how soon all of its loads are in flight and by VALU issue, not by
// bandwidth.  With v_dot4 every 4 multiply-adds cost a VALU slot; with
// v_mfma_i32_32x32x32_i8 a wave spends ONE instruction on 32 rows x 32 values
// and the VALU only unpacks nibbles and applies scales.  The batch rides along
// for free: the MFMA's other operand holds up to 32 activation rows.
//
// Work decomposition
//   * a workgroup owns 32 consecutive output rows; its waves split K into
//     slices of BPW 256-value blocks (K = 5120: 4 waves x 5 blocks);
//   * lane l = (n = l % 32, g = l / 32) loads, for each of its BPW blocks, the
//     16-byte header of row n and the four 16-byte nibble chunks
//     [32*j + 16*g, +16), j = 0..3: exactly the B operand of the MFMA for the
//     sub-block pair (2j, 2j+1), K positions 16*g..16*g+15.  All 5*BPW loads of
//     a wave are issued before anything else, so the whole matrix is in flight
//     at once across the chip;
//   * meanwhile the workgroup quantizes the activations to q8_1 into LDS (their
//     loads are issued before the weight loads, because the memory counter
//     retires in order);
//   * per sub-block: A = int8 activations of batch row (lane % 32) from LDS
//     (zero for rows >= batch), B = unpacked nibbles, zero accumulator input.
//     The result tile has the batch row in the register index: lane (n, g)
//     register v holds batch row 4*g + v of output row n for v < 4, so a batch
//     of 1..4 costs VB = 1..4 epilogue chains per sub-block and lanes g = 1
//     carry batch rows 4..7;
//   * epilogue per used register: t = (d*sc) * float(dot), acc = fma(xd, t, acc),
//     acc = fma(-dmin*mn, xd*qsum, acc)
//     (the arithmetic of gguf_q4_k_gemv.hip:893-904);
//   * K slices are summed through LDS in slice order.
#pragma once

#include "gguf_gemv_run.hpp"

namespace hipengine_gfx950 {

typedef int gm_v4i __attribute__((ext_vector_type(4)));
typedef int gm_v16i __attribute__((ext_vector_type(16)));
typedef uint32_t gm_u32x4 __attribute__((ext_vector_type(4)));

struct GemvMfmaArgs {
  const void* x;
  const uint8_t* w;
  void* out;
  int x_kind;
  int out_kind;
  int rows;    // batch rows, 1..B
  int K;
  int N;
  int waves;   // waves per workgroup = K slices
};

// LDS: the padded q8_1 image of gguf_gemv_run.hpp (B rows), one zero block for
// the unused A rows, and the K-slice partial sums.
inline size_t gemv_mfma_lds_bytes(int B, int K, int waves) {
  return gemv_run_lds_bytes(GGML_Q4_K, B, K) + 32 + static_cast<size_t>(waves) * 8 * 32 * 4;
}

template <int B, int BPW, int S>
__device__ __forceinline__ void gemv_mfma_q4k_workgroup(const GemvMfmaArgs& a, uint8_t* smem) {
  constexpr int Q8S = run_q8_stride<GGML_Q4_K>();
  constexpr int VB = B < 4 ? B : 4;                 // result registers in use per lane
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n = lane & 31, g = lane >> 5;
  const int nb = a.K / QK_K;
  const int row = min(static_cast<int>(blockIdx.x) * 32 + n, a.N - 1);
  const int kb0 = wave * BPW;

  uint8_t* q8 = smem;
  float* rec = reinterpret_cast<float*>(q8 + B * nb * Q8S);
  int* s16 = reinterpret_cast<int*>(rec + B * nb * 16);           // unused for Q4_K, same address as zero pad
  uint8_t* zero = reinterpret_cast<uint8_t*>(rec + B * nb * 16);  // 32 bytes of zeros
  float* red = reinterpret_cast<float*>(zero + 32);               // [waves][8][32]

  // activation loads first, then every weight load of this wave
  const GemvRunArgs ra{a.x, a.w, a.out, a.x_kind, a.out_kind, a.rows, a.K, a.N, a.waves};
  StageRegs<B, S> sr;
  gemv_run_stage_fetch<GGML_Q4_K, B, S>(ra, sr);

  gm_u32x4 hd[BPW], wq[BPW][4];
  const uint8_t* wrow = a.w + static_cast<int64_t>(row) * nb * Q4_K_BYTES;
#pragma unroll
  for (int c = 0; c < BPW; ++c) {
    const uint8_t* p = wrow + static_cast<int64_t>(min(kb0 + c, nb - 1)) * Q4_K_BYTES;
    hd[c] = *reinterpret_cast<const gm_u32x4*>(p);
#pragma unroll
    for (int j = 0; j < 4; ++j) wq[c][j] = *reinterpret_cast<const gm_u32x4*>(p + 16 + 32 * j + 16 * g);
  }

  if (tid < 8) reinterpret_cast<uint32_t*>(zero)[tid] = 0u;
  gemv_run_stage_commit<GGML_Q4_K, B, S>(ra, sr, q8, rec, s16);
  __syncthreads();

  float acc[VB];
#pragma unroll
  for (int v = 0; v < VB; ++v) acc[v] = 0.0f;

  // A operand address: batch row (lane % 32) when it exists, else the zero block
  const bool has_row = n < a.rows;
  const uint8_t* a_base = has_row ? q8 + n * nb * Q8S + 16 * g : zero;
  const int a_mul = has_row ? 1 : 0;
  // scale records of the batch rows this lane's result registers belong to
  const float* rec_g = rec + min(4 * g, B - 1) * nb * 16;

#pragma unroll
  for (int c = 0; c < BPW; ++c) {
    const int kb = kb0 + c;
    const bool live = kb < nb;
    const int kbc = min(kb, nb - 1);
    const Q4KScales u = q4k_unpack_scales(hd[c].y, hd[c].z, hd[c].w);
    float d = f16_bits_to_float(hd[c].x & 0xFFFFu);
    float dmin = f16_bits_to_float(hd[c].x >> 16);
    d = live ? d : 0.0f;
    dmin = live ? dmin : 0.0f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const gm_u32x4 qs = wq[c][j];
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        const int sb = 2 * j + half;
        const gm_v4i wop = half == 0
            ? gm_v4i{static_cast<int>(q4k_low(qs.x)), static_cast<int>(q4k_low(qs.y)),
                     static_cast<int>(q4k_low(qs.z)), static_cast<int>(q4k_low(qs.w))}
            : gm_v4i{static_cast<int>(q4k_high(qs.x)), static_cast<int>(q4k_high(qs.y)),
                     static_cast<int>(q4k_high(qs.z)), static_cast<int>(q4k_high(qs.w))};
        const gm_v4i xop = *reinterpret_cast<const gm_v4i*>(a_base + a_mul * (kbc * Q8S + sb * 32));
        gm_v16i c0;
#pragma unroll
        for (int v = 0; v < 16; ++v) c0[v] = 0;
        const gm_v16i dots = __builtin_amdgcn_mfma_i32_32x32x32_i8(xop, wop, c0, 0, 0, 0);
        const uint32_t sc = ((sb < 4 ? u.sc_lo : u.sc_hi) >> (8 * (sb & 3))) & 0xFFu;
        const uint32_t mn = ((sb < 4 ? u.mn_lo : u.mn_hi) >> (8 * (sb & 3))) & 0xFFu;
        const float sw = d * static_cast<float>(sc);
        const float mw = -(dmin * static_cast<float>(mn));
#pragma unroll
        for (int v = 0; v < VB; ++v) {
          // record of batch row 4*g + v: {xd(2j), xd(2j+1), xd*qsum(2j), xd*qsum(2j+1)} at [kb*16 + j*4]
          const float* r = rec_g + min(v, B - 1 - min(4 * g, B - 1)) * nb * 16 + kbc * 16 + j * 4;
          const float xd = r[half], xs = r[2 + half];
          const float t = sw * static_cast<float>(dots[v]);      // d*sc*dot, one rounding (|dot| < 2^24)
          acc[v] = __builtin_fmaf(xd, t, acc[v]);
          acc[v] = __builtin_fmaf(mw, xs, acc[v]);
        }
      }
    }
  }

  // K-slice reduction: red[wave][batch row][n]
#pragma unroll
  for (int v = 0; v < VB; ++v) {
    const int m = 4 * g + v;
    if (m < B) red[(wave * 8 + m) * 32 + n] = acc[v];
  }
  __syncthreads();
  for (int idx = tid; idx < B * 32; idx += blockDim.x) {
    const int m = idx >> 5, nn = idx & 31;
    const int orow = static_cast<int>(blockIdx.x) * 32 + nn;
    if (m < a.rows && orow < a.N) {
      float v = 0.0f;
      for (int s = 0; s < a.waves; ++s) v += red[(s * 8 + m) * 32 + nn];
      store_scalar(a.out, static_cast<int64_t>(m) * a.N + orow, v, a.out_kind);
    }
  }
}

}  // namespace hipengine_gfx950
