// Tile engine of the Q8_0 x D4S4 MMQ GEMM on the gfx950 int8 MFMA, shared by the dense prefill GEMM and the
// expert-grouped (MoE) GEMM.
//
//   out[m,n] = sum_{32-value block b} xd_b[m] * d_b[n] * dot_b[m,n]
//   (the weight is d * q per 34-byte block {half d; int8 qs[32]}, kernels/hip_gfx1100/quant/gguf_k_gemv.hip:98-105;
//   the activation xd * q per 32 values of a D4S4 block, gguf_k_mmq_prefill.hip:655-664)
//
// The plan of the Q6_K engine (gguf_mmq_q6k.hpp): 256 threads = 4 waves on a 128 x COLS output tile, one 128-value
// K step at a time (one D4S4 block per row, four Q8_0 blocks = 136 bytes per column), global -> registers (the
// next step's loads issued before this step is computed) -> LDS -> MFMA operands.  The weights are int8 already, so
// staging only separates the four scales from the values; one v_mfma_i32_32x32x32_i8 spans exactly one block, and
// its int32 result takes the two FMAs of the other engines (d * dot rounded once, then the activation scale).
#pragma once

#include "gguf_mmq_q6k.hpp"

namespace hipengine_gfx950 {

constexpr int Q8_0_STEP_BYTES = 4 * Q8_0_BYTES;   // weight bytes of one column and K step

template <int COLS>
struct Q8Smem {
  uint8_t xa[Q6_BM * A6_STRIDE];
  uint8_t w8[COLS * W6_STRIDE];   // 128 int8 values per column, padded to 9 x 16 B
  float sw[4][COLS];              // d of the step's four blocks, by column
  float cw[4][COLS];              // -MMQ_MAGIC * d (exact: d has 11 significant bits)
  float xd[4][Q6_BM];             // activation scale per 32 values, by row
};

struct Q8StepRegs {
  u32x4 pa[5];      // 128 rows x 10 chunks = 1280 = 5 per thread
  u32x4 q[2][2];    // threads 0..2*COLS-1: the 32 values of blocks 2*(tid&1) and 2*(tid&1)+1 of column tid/2
  uint32_t d[2];    //                      and their fp16 d's
  u32x4 xd;         // the last 128 threads: the four float scales of row tid - 128
};

template <int COLS, class RowOf, class ColOf>
__device__ __forceinline__ void q8_step_load(const uint8_t* xq, const uint8_t* w, int step, int64_t w_row_bytes,
                                             int64_t x_row_bytes, int tid, RowOf row_of, ColOf col_of,
                                             Q8StepRegs& r) {
#pragma unroll
  for (int i = 0; i < 5; ++i) {
    const int c = tid + i * Q6_THREADS;
    const int row = c / 10, part = c - row * 10;
    r.pa[i] = *reinterpret_cast<const u32x4*>(xq + row_of(row) * x_row_bytes + static_cast<int64_t>(step) * D4S4_BYTES +
                                              part * 16);
  }
  if (tid < 2 * COLS) {
    const uint8_t* blk = w + col_of(tid >> 1) * w_row_bytes + static_cast<int64_t>(step) * Q8_0_STEP_BYTES +
                         (tid & 1) * 2 * Q8_0_BYTES;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const uint4 lo = load16(blk + j * Q8_0_BYTES + 2), hi = load16(blk + j * Q8_0_BYTES + 18);
      r.q[j][0] = u32x4{lo.x, lo.y, lo.z, lo.w};
      r.q[j][1] = u32x4{hi.x, hi.y, hi.z, hi.w};
      r.d[j] = load2(blk + j * Q8_0_BYTES);
    }
  }
  if (tid >= Q6_THREADS - Q6_BM) {
    r.xd = *reinterpret_cast<const u32x4*>(xq + row_of(tid - (Q6_THREADS - Q6_BM)) * x_row_bytes +
                                           static_cast<int64_t>(step) * D4S4_BYTES);
  }
}

template <int COLS>
__device__ __forceinline__ void q8_step_store(Q8Smem<COLS>& s, int tid, const Q8StepRegs& r) {
#pragma unroll
  for (int i = 0; i < 5; ++i) {
    const int c = tid + i * Q6_THREADS;
    const int row = c / 10, part = c - row * 10;
    *reinterpret_cast<u32x4*>(s.xa + row * A6_STRIDE + part * 16) = r.pa[i];
  }
  if (tid < 2 * COLS) {
    const int col = tid >> 1, b0 = (tid & 1) * 2;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      uint8_t* dst = s.w8 + col * W6_STRIDE + (b0 + j) * 32;
      *reinterpret_cast<u32x4*>(dst) = r.q[j][0];
      *reinterpret_cast<u32x4*>(dst + 16) = r.q[j][1];
      const float d = f16_bits_to_float(r.d[j] & 0xFFFFu);
      s.sw[b0 + j][col] = d;
      s.cw[b0 + j][col] = -MMQ_MAGIC * d;
    }
  }
  if (tid >= Q6_THREADS - Q6_BM) {
#pragma unroll
    for (int j = 0; j < 4; ++j) s.xd[j][tid - (Q6_THREADS - Q6_BM)] = bits_to_float(r.xd[j]);
  }
}

// The whole K loop of one 128 x COLS output tile on 256 threads.  `emit(row, col, value)` receives every element
// of the tile (tile-relative coordinates) once; with DUMP, `dump(row, col, block, dot)` receives every int32
// block dot (block = index of the 32 values along K).  `steps` = K / 128.
template <bool DUMP, int COLS, class RowOf, class ColOf, class Emit, class Dump = int>
__device__ __forceinline__ void q8_tile_run(const uint8_t* xq, int64_t x_row_bytes, const uint8_t* w, int64_t w_row_bytes,
                                            int steps, Q8Smem<COLS>& s, RowOf row_of, ColOf col_of, Emit emit,
                                            Dump dump = 0) {
  static_assert(COLS == 128 || COLS == 64, "two wave columns of one or two 32-wide tiles");
  constexpr int NT = COLS / 64;                   // 32-wide n tiles per wave
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave & 1, wn = wave >> 1;
  const int lc = lane & 31, g = lane >> 5;

  float acc[NT][2][16];
#pragma unroll
  for (int i = 0; i < NT; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  Q8StepRegs regs;
  q8_step_load<COLS>(xq, w, 0, w_row_bytes, x_row_bytes, tid, row_of, col_of, regs);

  for (int step = 0; step < steps; ++step) {
    q8_step_store(s, tid, regs);
    __syncthreads();
    if (step + 1 < steps) q8_step_load<COLS>(xq, w, step + 1, w_row_bytes, x_row_bytes, tid, row_of, col_of, regs);

    v16i ci;
#pragma unroll
    for (int v = 0; v < 16; ++v) ci[v] = static_cast<int>(MMQ_MAGIC_BITS);
#pragma unroll
    for (int sl = 0; sl < 4; ++sl) {            // one 32-value block of the weights, one activation scale
      v4i wop[NT], xop[2];
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
        wop[nt] = *reinterpret_cast<const v4i*>(s.w8 + (wn * 32 * NT + nt * 32 + lc) * W6_STRIDE + 32 * sl + 16 * g);
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
        xop[mt] = *reinterpret_cast<const v4i*>(s.xa + (wm * 64 + mt * 32 + lc) * A6_STRIDE + 32 + 32 * sl + 16 * g);
      // Software pipeline over the 2 * NT (m tile, n tile) pairs: the MFMA of pair i+1 is issued before the
      // scale arithmetic of pair i.
      constexpr int PAIRS = 2 * NT;
      auto issue = [&](int i) {
        return __builtin_amdgcn_mfma_i32_32x32x32_i8(xop[i / NT], wop[i % NT], ci, 0, 0, 0);
      };
      v16i cur = issue(0);
#pragma unroll
      for (int i = 0; i < PAIRS; ++i) {
        const int mt = i / NT, nt = i % NT;
        v16i next = cur;
        if (i + 1 < PAIRS) next = issue(i + 1);
        float xdv[16];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float4 t = *reinterpret_cast<const float4*>(&s.xd[sl][wm * 64 + mt * 32 + 8 * j + 4 * g]);
          xdv[4 * j] = t.x; xdv[4 * j + 1] = t.y; xdv[4 * j + 2] = t.z; xdv[4 * j + 3] = t.w;
        }
        const int col = wn * 32 * NT + nt * 32 + lc;
        if constexpr (DUMP) {
#pragma unroll
          for (int v = 0; v < 16; ++v)
            dump(wm * 64 + mt * 32 + 8 * (v >> 2) + 4 * g + (v & 3), col, step * 4 + sl,
                 cur[v] - static_cast<int>(MMQ_MAGIC_BITS));
        }
        const float sw = s.sw[sl][col], cw = s.cw[sl][col];
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const float t = __builtin_fmaf(bits_to_float(static_cast<uint32_t>(cur[v])), sw, cw);   // d * dot, rounded once
          acc[nt][mt][v] = __builtin_fmaf(xdv[v], t, acc[nt][mt][v]);
        }
        cur = next;
      }
    }
    __syncthreads();
  }

  // lane holds column lc of each n tile and rows 8*(v/4) + 4*g + v%4 of each m tile
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
      for (int v = 0; v < 16; ++v)
        emit(wm * 64 + mt * 32 + 8 * (v >> 2) + 4 * g + (v & 3), wn * 32 * NT + nt * 32 + lc, acc[nt][mt][v]);
}

}  // namespace hipengine_gfx950
