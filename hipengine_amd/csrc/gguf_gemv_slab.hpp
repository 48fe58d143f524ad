// "Slab" form of the q8_1 decode GEMV for Q4_K weights, batch 1..8, on the int8
// MFMA: one workgroup per CU owns a slab of consecutive output rows, its waves
// split K, and nothing in the kernel waits for another wave until the final sum.
//
// Why: with v_dot4 a batch of 8 costs eight times the VALU work of batch 1 and
// the kernel stops being bound by HBM.  v_mfma_i32_32x32x32_i8 takes 32 weight
// rows x 32 values against up to 32 activation rows in one instruction, so the
// batch rides along and the VALU only splits nibbles and applies scales.
//
// Work decomposition
//   * workgroup b owns rows [b*R, b*R + R), R = ceil(N / 256) <= 96, in steps of 32;
//   * wave w owns one or two consecutive K blocks of every row: the first `two_block_waves`
//     waves two, the others one (K = 5120: 12 waves = 8 x 2 + 4 x 1 blocks, which gives every
//     SIMD three waves and five blocks; 10 waves x 2 blocks would load two SIMDs with six).  It quantizes ONLY its own K slice of the
//     activations (B x BPW x 256 values) into wave-private LDS: no workgroup
//     barrier before the final sum;
//   * per step the wave reads its 32 x (BPW*144) byte piece of the weight with
//     loads that are contiguous along each row (lane c takes 16-byte chunk c of
//     the piece: BPW*9 chunks per row), writes the registers to wave-private LDS
//     in that natural order and reads them back in MFMA operand order: lane
//     (n = l % 32, g = l / 32) takes bytes [16 + 32j + 16g, +16) of row n, the
//     values 16g..16g+15 of sub-blocks 2j (low nibbles) and 2j+1 (high nibbles).
//     Loading in operand order directly would make every lane of a load touch a
//     different row (2880 bytes apart), which the texture addresser serializes;
//     The loads are unconditional: rows past the slab and chunks past the piece are
//     clamped to valid addresses and their bytes land in rows whose results are
//     dropped (or in a dump slot), which keeps the issue code free of branches;
//   * the loads of step t+1 are issued into step t's registers as soon as those are in
//     LDS and fly while step t is computed;
//   * A = int8 activations of batch row (l % 32) (zero for rows >= batch), B = the
//     nibbles, zero accumulator input.  Lane (n, g) register v < 4 of the result
//     is batch row 4g + v of output row n; per sub-block and batch row
//     t = (d*sc) * float(dot), acc = fma(xd, t, acc), acc = fma(-dmin*mn, xd*qsum, acc)
//     (the arithmetic of gguf_q4_k_gemv.hip:893-904);
//   * K slices are summed through LDS in slice order.
//
// LDS row pitch: 144 bytes (BPW = 1) or 304 (BPW = 2), i.e. 4 x an odd number of
// dwords, which puts the 16-byte operand reads of 16 consecutive rows on
// distinct banks.
#pragma once

#include "gguf_gemv_run.hpp"

namespace hipengine_gfx950 {

typedef int sl_v4i __attribute__((ext_vector_type(4)));
typedef int sl_v16i __attribute__((ext_vector_type(16)));
typedef uint32_t sl_u32x4 __attribute__((ext_vector_type(4)));
typedef float sl_f4 __attribute__((ext_vector_type(4)));

struct GemvSlabArgs {
  const void* x;
  const uint8_t* w;
  void* out;
  int x_kind;
  int out_kind;
  int rows;      // batch rows, 1..B
  int K;
  int N;
  int rows_wg;   // output rows per workgroup, 1..96
  int waves;     // waves per workgroup
  int two_block_waves;   // waves 0..two_block_waves-1 own two K blocks each, the rest one
  const void* residual;   // null, or [rows, N] of the output type: out = round(projection) + residual
  const void* gate;       // null, or [rows, N] of the output type (may be `out` itself): out = silu(gate) * round(projection)
  const uint8_t* w_up;    // pair kernels only: the second matrix (w is the gate), out = silu(round(gate.x)) * round(up.x)
  int32_t* dots_out;      // verification kernels only: int32 [rows, N, K/32], every sub-block dot as the MFMA returns it
};

constexpr int SLAB_MAX_ROWS = 96;
constexpr int SLAB_MAX_MATRICES = 4;

// Several matrices over one activation in one launch: workgroups [wg_end[i-1], wg_end[i]) take matrix i
// (its own row count, rows per workgroup, weight and output; the same K, batch and layout).
struct GemvSlabMultiArgs {
  GemvSlabArgs sub[SLAB_MAX_MATRICES];
  int wg_end[SLAB_MAX_MATRICES];
  int count;
};
constexpr int SLAB_MAX_PAIR_ROWS = 72;   // rows per workgroup and matrix of the pair kernels: 2 x 72 partial sums per batch row

template <int BPW>
constexpr int slab_row_pitch() { return BPW == 1 ? 144 : 304; }

// Per wave of `blocks` (1 or 2) K blocks: the weight piece of a step (reused for the partial sums
// after the last step), a 16-byte dump slot, the scale records and the int8 activations.
constexpr int slab_pitch(int blocks) { return blocks == 1 ? 144 : 304; }
constexpr int slab_wave_bytes(int B, int blocks) {
  return 32 * slab_pitch(blocks) + 16 + blocks * 8 * 16 * 4 + B * (blocks * 256 + 16);
}

inline size_t gemv_slab_lds_bytes(int b, int waves, int two_block_waves) {
  return static_cast<size_t>(two_block_waves) * slab_wave_bytes(b, 2) +
         static_cast<size_t>(waves - two_block_waves) * slab_wave_bytes(b, 1);
}

// VERIFY: the verification instantiation, which also writes every int32 sub-block dot to a.dots_out.
// PAIR: the workgroup walks its rows of the gate matrix (a.w), then the same rows of the up matrix (a.w_up), and
// stores silu(round(gate)) * round(up): the arithmetic of a gate launch followed by an up launch with a.gate set,
// in one launch (one staging of the activations, no round trip of the gate through memory).
// `wg`: the workgroup's index among those of this matrix (the multi-matrix kernel hands every matrix a range).
template <int B, int BPW, int XK, bool VERIFY = false, bool PAIR = false>
__device__ __forceinline__ void gemv_slab_q4k_workgroup(const GemvSlabArgs& a, uint8_t* smem, int wg) {
  static_assert(!(PAIR && VERIFY), "the verification kernel takes one matrix");
  constexpr int VB = B < 4 ? B : 4;                  // result registers in use per lane
  constexpr int NL = (32 * BPW * 9 + 63) / 64;       // 16-byte loads per lane and step
  constexpr int NM = PAIR ? 2 : 1;                   // matrices
  constexpr int STEPS_PER = SLAB_MAX_ROWS / 32;      // steps per matrix
  constexpr int MAX_STEPS = NM * STEPS_PER;
  constexpr int RED_ROWS = PAIR ? 2 * SLAB_MAX_PAIR_ROWS : SLAB_MAX_ROWS;   // partial sums per batch row
  constexpr int EARLY_TAIL_ROWS = 7;                 // a last step of at most this many rows is done first
  constexpr int NLT = (EARLY_TAIL_ROWS * BPW * 9 + 63) / 64;
  static_assert(B * RED_ROWS * 4 <= 32 * slab_pitch(1), "partial sums must fit the weight piece");
  const int x_kind = XK >= 0 ? XK : a.x_kind;

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 31, g = lane >> 5;
  const int nb = a.K / QK_K;
  const int t2 = BPW == 2 ? a.two_block_waves : 0;
  const int blocks_w = wave < t2 ? 2 : 1;
  const int kb0 = wave < t2 ? 2 * wave : t2 + wave;
  // LDS layout of this wave (sizes depend on its block count)
  const int PITCH = slab_pitch(blocks_w);
  const int XQ_PITCH = blocks_w * 256 + 16;            // int8 activations, one batch row
  const int DUMP = 32 * PITCH;
  const int REC = DUMP + 16;
  const int XQ = REC + blocks_w * 8 * 16 * 4;
  const int wave_off = wave < t2 ? wave * slab_wave_bytes(B, 2)
                                 : t2 * slab_wave_bytes(B, 2) + (wave - t2) * slab_wave_bytes(B, 1);
  const int r0 = wg * a.rows_wg;
  const int rows_wg = min(a.rows_wg, a.N - r0);
  const int steps = (rows_wg + 31) >> 5;
  const int row_bytes = nb * Q4_K_BYTES;
  const int64_t wg_offset = static_cast<int64_t>(r0) * row_bytes + kb0 * Q4_K_BYTES;

  uint8_t* wq = smem + wave_off;
  float* rec = reinterpret_cast<float*>(wq + REC);   // [BPW*8 sub-blocks][xd[8], xd*qsum[8]]
  uint8_t* xq = wq + XQ;

  // ---- activation loads of this wave's K slice: 4 lanes per 32-value group, 8 values per lane,
  // 16 groups per pass.  Group p*16 + quad is batch row gid / (blocks_w*8), sub-block gid % (blocks_w*8);
  // a one-block wave is done after half the passes of a two-block wave.
  constexpr int PASSES = (B * BPW * 8 + 15) / 16;
  const int gshift = blocks_w == 2 ? 4 : 3;
  const int passes = (B * blocks_w * 8 + 15) >> 4;
  const int quad = lane >> 2, e = lane & 3;
  uint32_t raw[PASSES][8];
#pragma unroll
  for (int p = 0; p < PASSES; ++p) {
    const int gid = p * 16 + quad;
    // clamped, unconditional: rows >= a.rows and blocks past the slice are quantized but not used
    const int bb = min(gid >> gshift, a.rows - 1);
    const int rem = gid & ((1 << gshift) - 1);
    const int j = (kb0 + (rem >> 3)) * 8 + (rem & 7);
#pragma unroll
    for (int i = 0; i < 8; ++i) raw[p][i] = 0u;
    if (p >= passes) {
      // nothing left for this wave
    } else if (x_kind == KIND_F32) {
      const uint4* src = reinterpret_cast<const uint4*>(static_cast<const float*>(a.x) + static_cast<int64_t>(bb) * a.K + j * 32 + e * 8);
      const uint4 lo = src[0], hi = src[1];
      raw[p][0] = lo.x; raw[p][1] = lo.y; raw[p][2] = lo.z; raw[p][3] = lo.w;
      raw[p][4] = hi.x; raw[p][5] = hi.y; raw[p][6] = hi.z; raw[p][7] = hi.w;
    } else if (x_kind == KIND_Q8_1) {
      const uint8_t* blk = static_cast<const uint8_t*>(a.x) + (static_cast<int64_t>(bb) * (a.K / 32) + j) * Q8_1_BYTES;
      raw[p][0] = *reinterpret_cast<const uint32_t*>(blk + 4 + 8 * e);
      raw[p][1] = *reinterpret_cast<const uint32_t*>(blk + 8 + 8 * e);
      raw[p][2] = *reinterpret_cast<const uint32_t*>(blk);
    } else {
      const uint4 h = *reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(a.x) + static_cast<int64_t>(bb) * a.K + j * 32 + e * 8);
      raw[p][0] = h.x; raw[p][1] = h.y; raw[p][2] = h.z; raw[p][3] = h.w;
    }
  }

  // ---- chunk c = i*64 + lane of a step's piece: row c / cpr, 16-byte column c % cpr
  const int cpr = blocks_w * 9;
  const int row_inc = (BPW == 2 && cpr == 18) ? 3 : 7, col_inc = (BPW == 2 && cpr == 18) ? 10 : 1;   // 64 = row_inc*cpr + col_inc
  // The positions are walked again from (row0, col0) wherever they are needed (four
  // operations per chunk) instead of being kept in NL registers.
  const int row0 = (BPW == 2 && cpr == 18) ? lane / 18 : lane / 9;
  const int col0 = lane - row0 * cpr;
  auto walk = [&](auto&& visit) {
    int row = row0, col = col0;
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      visit(i, row, col * 16);
      row += row_inc; col += col_inc;
      if (col >= cpr) { col -= cpr; row += 1; }
    }
  };

  sl_u32x4 buf[NL];
  // Buffer loads: a descriptor over this wave's K slice of the slab (the hardware returns
  // zeros past its end), a 32-bit lane offset and a scalar step offset: no 64-bit
  // address arithmetic per load.
  const int slab_bytes = (rows_wg - 1) * row_bytes + blocks_w * Q4_K_BYTES;
  const __amdgpu_buffer_rsrc_t wrsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint8_t*>(a.w + wg_offset), 0, slab_bytes, 0x00020000);
  // the pair kernels' second matrix (the same slab of rows of a.w_up)
  const __amdgpu_buffer_rsrc_t wrsrc_up = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint8_t*>((PAIR ? a.w_up : a.w) + wg_offset), 0, slab_bytes, 0x00020000);
  // step t of matrix m
  auto issue = [&](int m, int t, sl_u32x4 (&dst)[NL]) {
    const int last = rows_wg - 32 * t - 1;           // >= 0 for t < steps
    if (PAIR && m) {
      walk([&](int i, int row, int col16) {
        dst[i] = __builtin_amdgcn_raw_buffer_load_b128(wrsrc_up, min(row, last) * row_bytes + col16, t * 32 * row_bytes, 0);
      });
    } else {
      walk([&](int i, int row, int col16) {
        dst[i] = __builtin_amdgcn_raw_buffer_load_b128(wrsrc, min(row, last) * row_bytes + col16, t * 32 * row_bytes, 0);
      });
    }
  };
  // A short last step (N = 17408: 68 rows per slab = 32 + 32 + 4) is loaded up front into its own
  // few registers and computed first, while the first full step is still on its way; done
  // last, it would cost a whole step of MFMA and scale work with nothing left to overlap.
  const int tail_rows = rows_wg & 31;
  const bool early_tail = steps > 1 && tail_rows >= 1 && tail_rows <= EARLY_TAIL_ROWS;
  sl_u32x4 tbuf[NM][NLT];
  if (early_tail) {
    walk([&](int i, int row, int col16) {
      if (i < NLT) {
        tbuf[0][i] = __builtin_amdgcn_raw_buffer_load_b128(wrsrc, min(row, tail_rows - 1) * row_bytes + col16,
                                                           (steps - 1) * 32 * row_bytes, 0);
        if constexpr (PAIR)
          tbuf[1][i] = __builtin_amdgcn_raw_buffer_load_b128(wrsrc_up, min(row, tail_rows - 1) * row_bytes + col16,
                                                             (steps - 1) * 32 * row_bytes, 0);
      }
    });
  }
  // batch 8 holds 64 registers of fetched activations: its first weight loads wait until half of
  // them are quantized (they are not needed before the staging is done)
  if constexpr (B < 8) issue(0, 0, buf);

  // ---- quantize the slice into LDS
#pragma unroll
  for (int p = 0; p < PASSES; ++p) {
    if constexpr (B >= 8) {
      if (p == PASSES / 2) issue(0, 0, buf);
    }
    if (p >= passes) continue;
    const int gid = p * 16 + quad;
    const int b = gid >> gshift, rem = gid & ((1 << gshift) - 1);
    uint32_t packed[2];
    float xd;
    q8_quantize8(x_kind, raw[p], true, packed, xd);
    const bool used = b < a.rows;
    packed[0] = used ? packed[0] : 0u;
    packed[1] = used ? packed[1] : 0u;
    xd = used ? xd : 0.0f;
    int total = dot4(0x01010101u, packed[1], dot4(0x01010101u, packed[0], 0));
    total += dpp_i<DPP_QUAD_XOR1>(total);
    total += dpp_i<DPP_QUAD_XOR2>(total);
    if (b < B) {
      *reinterpret_cast<uint2*>(xq + b * XQ_PITCH + rem * 32 + e * 8) = make_uint2(packed[0], packed[1]);
      if (e == 0) {
        rec[rem * 16 + b] = xd;
        rec[rem * 16 + 8 + b] = xd * static_cast<float>(total);
      }
    }
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

  // partial sums of the steps done so far, filed with selects (the step loop is a real loop)
  float done[MAX_STEPS][VB];
#pragma unroll
  for (int t = 0; t < MAX_STEPS; ++t)
#pragma unroll
    for (int v = 0; v < VB; ++v) done[t][v] = 0.0f;

  const uint8_t* wlane = wq + n * PITCH;
  const uint8_t* alane = xq + min(n, B - 1) * XQ_PITCH + 16 * g;   // A operand row: batch row n (zeros for n >= B)
  const sl_f4* rec4 = reinterpret_cast<const sl_f4*>(rec);

  auto to_lds = [&](const sl_u32x4 (&src)[NL]) {
    walk([&](int i, int row, int col16) {
      *reinterpret_cast<sl_u32x4*>(wq + (row < 32 ? row * PITCH + col16 : DUMP)) = src[i];
    });
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  };

  // `slot` = matrix * STEPS_PER + step: where the result is filed
  auto compute = [&](int slot) {
    const int t = slot;     // the verification kernel has one matrix
    float acc[VB];
#pragma unroll
    for (int v = 0; v < VB; ++v) acc[v] = 0.0f;
#pragma unroll
    for (int s = 0; s < BPW; ++s) {
      if (s < blocks_w) {
        const sl_u32x4 hd = *reinterpret_cast<const sl_u32x4*>(wlane + s * Q4_K_BYTES);
        const Q4KScales u = q4k_unpack_scales(hd.y, hd.z, hd.w);
        const float d = f16_bits_to_float(hd.x & 0xFFFFu);
        const float dmin = f16_bits_to_float(hd.x >> 16);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const sl_u32x4 qs = *reinterpret_cast<const sl_u32x4*>(wlane + s * Q4_K_BYTES + 16 + 32 * j + 16 * g);
#pragma unroll
          for (int half = 0; half < 2; ++half) {
            const int sb = 2 * j + half;
            const sl_v4i wop = half == 0
                ? sl_v4i{static_cast<int>(q4k_low(qs.x)), static_cast<int>(q4k_low(qs.y)),
                         static_cast<int>(q4k_low(qs.z)), static_cast<int>(q4k_low(qs.w))}
                : sl_v4i{static_cast<int>(q4k_high(qs.x)), static_cast<int>(q4k_high(qs.y)),
                         static_cast<int>(q4k_high(qs.z)), static_cast<int>(q4k_high(qs.w))};
            sl_v4i xop = sl_v4i{0, 0, 0, 0};
            xop = *reinterpret_cast<const sl_v4i*>(alane + s * 256 + sb * 32);
            sl_v16i c0;
#pragma unroll
            for (int v = 0; v < 16; ++v) c0[v] = 0;
            const sl_v16i dots = __builtin_amdgcn_mfma_i32_32x32x32_i8(xop, wop, c0, 0, 0, 0);
            if constexpr (VERIFY) {
              const int row = 32 * t + n;
#pragma unroll
              for (int v = 0; v < VB; ++v) {
                const int m = 4 * g + v;
                if (m < a.rows && row < rows_wg)
                  a.dots_out[(static_cast<int64_t>(m) * a.N + r0 + row) * (a.K / 32) + (kb0 + s) * 8 + sb] = dots[v];
              }
            }
            const uint32_t sc = ((sb < 4 ? u.sc_lo : u.sc_hi) >> (8 * (sb & 3))) & 0xFFu;
            const uint32_t mn = ((sb < 4 ? u.mn_lo : u.mn_hi) >> (8 * (sb & 3))) & 0xFFu;
            const float sw = d * static_cast<float>(sc);
            const float mw = -(dmin * static_cast<float>(mn));
            // scales of batch rows 4g..4g+VB-1: read only what the batch uses
            float xd[VB], xs[VB];
            if constexpr (VB == 4) {
              const sl_f4 d4 = rec4[(s * 8 + sb) * 4 + g], s4 = rec4[(s * 8 + sb) * 4 + 2 + g];
#pragma unroll
              for (int v = 0; v < 4; ++v) { xd[v] = d4[v]; xs[v] = s4[v]; }
            } else {
#pragma unroll
              for (int v = 0; v < VB; ++v) { xd[v] = rec[(s * 8 + sb) * 16 + v]; xs[v] = rec[(s * 8 + sb) * 16 + 8 + v]; }
            }
#pragma unroll
            for (int v = 0; v < VB; ++v) {
              const float tv = sw * static_cast<float>(dots[v]);   // |dot| < 2^24: one rounding
              acc[v] = __builtin_fmaf(xd[v], tv, acc[v]);
              acc[v] = __builtin_fmaf(mw, xs[v], acc[v]);
            }
          }
        }
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int u = 0; u < MAX_STEPS; ++u)
#pragma unroll
      for (int v = 0; v < VB; ++v) done[u][v] = (u == slot) ? acc[v] : done[u][v];
  };

  // the full steps of the matrices in turn: q = matrix * full_steps + step
  const int full_steps = early_tail ? steps - 1 : steps;
  const int nfull = NM * full_steps;
#pragma unroll 1
  for (int q = early_tail ? -NM : 0; q < nfull; ++q) {
    if (q < 0) {
      const int mt = q + NM;     // the short last step of matrix mt
      walk([&](int i, int row, int col16) {
        if (i < NLT) *reinterpret_cast<sl_u32x4*>(wq + row * PITCH + col16) = (PAIR && mt) ? tbuf[NM - 1][i] : tbuf[0][i];   // rows 0..7
      });
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    } else {
      to_lds(buf);
      const int qn = q + 1;
      if (qn < nfull) issue(qn >= full_steps, qn >= full_steps ? qn - full_steps : qn, buf);
    }
    compute(q < 0 ? (q + NM) * STEPS_PER + steps - 1 : q >= full_steps ? STEPS_PER + q - full_steps : q);
  }

  // ---- K-slice reduction: each wave's partial sums [batch row][RED_ROWS] replace its weight piece
  // (pair kernels: the rows of the up matrix follow the rows_wg rows of the gate matrix)
  float* red = reinterpret_cast<float*>(wq);
#pragma unroll
  for (int u = 0; u < MAX_STEPS; ++u) {
#pragma unroll
    for (int v = 0; v < VB; ++v) {
      const int m = 4 * g + v, rl = 32 * (u % STEPS_PER) + n;
      if (m < B && rl < rows_wg) red[m * RED_ROWS + (u / STEPS_PER) * rows_wg + rl] = done[u][v];
    }
  }
  __syncthreads();
  for (int idx = tid; idx < a.rows * rows_wg; idx += blockDim.x) {
    const int m = idx / rows_wg, rl = idx - m * rows_wg;
    float v = 0.0f, v_up = 0.0f;
    for (int s = 0; s < a.waves; ++s) {
      const int off = s < t2 ? s * slab_wave_bytes(B, 2) : t2 * slab_wave_bytes(B, 2) + (s - t2) * slab_wave_bytes(B, 1);
      v += reinterpret_cast<const float*>(smem + off)[m * RED_ROWS + rl];
      if constexpr (PAIR) v_up += reinterpret_cast<const float*>(smem + off)[m * RED_ROWS + rows_wg + rl];
    }
    const int64_t oi = static_cast<int64_t>(m) * a.N + r0 + rl;
    if constexpr (PAIR) {
      // what the gate launch stores and the up launch reads back and applies (gguf_q4_k_gemv.hip:652-657)
      const float gt = round_to_kind(v, a.out_kind);
      const float sig = 1.0f / (1.0f + expf(-gt));
      store_scalar(a.out, oi, gt * sig * round_to_kind(v_up, a.out_kind), a.out_kind);
      continue;
    }
    if (a.residual) v = round_to_kind(v, a.out_kind) + load_scalar(a.residual, oi, a.out_kind);
    if (a.gate) {   // the up half of a gate/up pair: the gate projection is already stored, rounded (gguf_q4_k_gemv.hip:652-657)
      const float gt = load_scalar(a.gate, oi, a.out_kind);
      const float sig = 1.0f / (1.0f + expf(-gt));
      v = gt * sig * round_to_kind(v, a.out_kind);
    }
    store_scalar(a.out, oi, v, a.out_kind);
  }
}

}  // namespace hipengine_gfx950
