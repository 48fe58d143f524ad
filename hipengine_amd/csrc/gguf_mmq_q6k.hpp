// Tile engine of the Q6_K x D4S4 MMQ GEMM on the gfx950 int8 MFMA, shared by the dense prefill GEMM and the
// expert-grouped (MoE) GEMM.
//
//   out[m,n] = sum_{32-wide group g} xd_g[m] * (s0*dot0 + s1*dot1),  s = d*scale_i8, dots over 16 values
//   (kernels/hip_gfx1100/quant/gguf_k_mmq_prefill.hip:652-667)
//
// 256 threads = 4 waves on a 128 x COLS output tile (COLS = 128: each wave 64 x 64 as 2 x 2 MFMA tiles of 32 x 32;
// COLS = 64: each wave 64 x 32), v_mfma_i32_32x32x16_i8 per 16 values, one 128-value K step at a time.
#pragma once

#include "gguf_mmq_q4k.hpp"

namespace hipengine_gfx950 {

constexpr int Q6_BM = 128, Q6_THREADS = 256;

// --------------------------------------------------------------------------
// Q6_K x D4S4.  One K step is 128 values: one D4S4 block per row and one half of
// a Q6_K block per column (64 ql bytes, 32 qh bytes, 8 int8 scales).  The 6-bit
// values are rebuilt and centred (u - 32) once per workgroup while the tile is
// written to LDS, so the waves read plain int8 MFMA operands on both sides.
// --------------------------------------------------------------------------
constexpr int A6_STRIDE = 176;   // 160-byte D4S4 block padded to 11 x 16 B
constexpr int W6_STRIDE = 144;   // 128 centred int8 values padded to 9 x 16 B

// COLS: columns of the workgroup's tile, 128 (each wave 64 x 64) or 64 (each wave 64 x 32: twice the tiles for
// a narrow N, whose 128-wide tiles leave a last round mostly empty).
template <int COLS>
struct Q6Smem {
  uint8_t xa[Q6_BM * A6_STRIDE];
  uint8_t w8[COLS * W6_STRIDE];
  float sw[8][COLS];   // d * scale of the 8 16-value groups of the step, by column
  float cw[8][COLS];   // -MMQ_MAGIC * sw (exact: d has 11 significant bits, the scale 8)
  float xd[4][Q6_BM];     // activation scale per 32 values, by row
};

struct Q6StepRegs {
  u32x4 pa[5];         // 128 rows x 10 chunks = 1280 = 5 per thread
  u32x4 qla, qlb, qh;  // 16 bytes each of the column tid/2, byte offset 16*(tid&1)
  uint2 sc;            // threads 0..COLS-1: the 8 scales of column tid
  uint32_t d;          //                    and its fp16 d
  u32x4 xd;            // threads COLS..COLS+127: the four float scales of row tid-COLS
};

// `row_of(r)` / `col_of(c)` give the activation row (in D4S4 blocks of x_row_bytes per row from xq) and the
// weight row (of w_row_bytes from w) that tile row r / tile column c read; rows and columns outside the
// problem are mapped to any valid one by the caller (their results are not stored).
template <int COLS, class RowOf, class ColOf>
__device__ __forceinline__ void q6_step_load(const uint8_t* xq, const uint8_t* w, int step, int64_t w_row_bytes,
                                             int64_t x_row_bytes, int tid, RowOf row_of, ColOf col_of,
                                             Q6StepRegs& r) {
  const int kb = step >> 1, hh = step & 1;
#pragma unroll
  for (int i = 0; i < 5; ++i) {
    const int c = tid + i * Q6_THREADS;
    const int row = c / 10, part = c - row * 10;
    r.pa[i] = *reinterpret_cast<const u32x4*>(xq + row_of(row) * x_row_bytes + static_cast<int64_t>(step) * D4S4_BYTES +
                                              part * 16);
  }
  if (tid < 2 * COLS) {
    const uint8_t* blk = w + col_of(tid >> 1) * w_row_bytes + static_cast<int64_t>(kb) * Q6_K_BYTES;
    const int o = (tid & 1) * 16;
    const uint4 x = load16(blk + 64 * hh + o), y = load16(blk + 64 * hh + 32 + o), z = load16(blk + 128 + 32 * hh + o);
    r.qla = u32x4{x.x, x.y, x.z, x.w};
    r.qlb = u32x4{y.x, y.y, y.z, y.w};
    r.qh = u32x4{z.x, z.y, z.z, z.w};
  }
  if (tid < COLS) {
    const uint8_t* blk = w + col_of(tid) * w_row_bytes + static_cast<int64_t>(kb) * Q6_K_BYTES;
    r.sc = load8(blk + 192 + 8 * hh);
    r.d = load2(blk + 208);
  } else if (tid < COLS + Q6_BM) {
    r.xd = *reinterpret_cast<const u32x4*>(xq + row_of(tid - COLS) * x_row_bytes +
                                           static_cast<int64_t>(step) * D4S4_BYTES);
  }
}

template <int COLS>
__device__ __forceinline__ void q6_step_store(Q6Smem<COLS>& s, int tid, const Q6StepRegs& r) {
#pragma unroll
  for (int i = 0; i < 5; ++i) {
    const int c = tid + i * Q6_THREADS;
    const int row = c / 10, part = c - row * 10;
    *reinterpret_cast<u32x4*>(s.xa + row * A6_STRIDE + part * 16) = r.pa[i];
  }
  if (tid < 2 * COLS) {
    u32x4 q0, q1, q2, q3;   // the four 32-value quarters of the half, bytes o..o+15 of each
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const Q6KQuad u = q6k_unpack(r.qla[i], r.qlb[i], r.qh[i]);
      q0[i] = q6k_center(u.g0); q1[i] = q6k_center(u.g1); q2[i] = q6k_center(u.g2); q3[i] = q6k_center(u.g3);
    }
    uint8_t* dst = s.w8 + (tid >> 1) * W6_STRIDE + (tid & 1) * 16;
    *reinterpret_cast<u32x4*>(dst) = q0;
    *reinterpret_cast<u32x4*>(dst + 32) = q1;
    *reinterpret_cast<u32x4*>(dst + 64) = q2;
    *reinterpret_cast<u32x4*>(dst + 96) = q3;
  }
  if (tid < COLS) {
    const float d = f16_bits_to_float(r.d & 0xFFFFu);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const uint32_t word = j < 4 ? r.sc.x : r.sc.y;
      const int sc = static_cast<int>(static_cast<int8_t>((word >> (8 * (j & 3))) & 0xFFu));
      const float sw = d * static_cast<float>(sc);
      s.sw[j][tid] = sw;
      s.cw[j][tid] = -MMQ_MAGIC * sw;
    }
  } else if (tid < COLS + Q6_BM) {
#pragma unroll
    for (int j = 0; j < 4; ++j) s.xd[j][tid - COLS] = bits_to_float(r.xd[j]);
  }
}

// The whole K loop of one 128 x COLS output tile on 256 threads.  `emit(row, col, value)` receives every element
// of the tile (tile-relative coordinates) once; with DUMP, `dump(row, col, group, dot)` receives every int32
// 16-value dot (group = index of the 16 values along K).
template <bool DUMP, int COLS, class RowOf, class ColOf, class Emit, class Dump = int>
__device__ __forceinline__ void q6_tile_run(const uint8_t* xq, int64_t x_row_bytes, const uint8_t* w, int64_t w_row_bytes,
                                            int steps, Q6Smem<COLS>& s, RowOf row_of, ColOf col_of, Emit emit,
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

  Q6StepRegs regs;
  q6_step_load<COLS>(xq, w, 0, w_row_bytes, x_row_bytes, tid, row_of, col_of, regs);

  for (int step = 0; step < steps; ++step) {
    q6_step_store(s, tid, regs);
    __syncthreads();
    if (step + 1 < steps) q6_step_load<COLS>(xq, w, step + 1, w_row_bytes, x_row_bytes, tid, row_of, col_of, regs);

    v16i ci;
#pragma unroll
    for (int v = 0; v < 16; ++v) ci[v] = static_cast<int>(MMQ_MAGIC_BITS);
#pragma unroll
    for (int sl = 0; sl < 4; ++sl) {            // 32 activation values share one scale
      long wop[NT][2];                           // [n tile][16-value group]
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int t = 0; t < 2; ++t)
          wop[nt][t] = *reinterpret_cast<const long*>(s.w8 + (wn * 32 * NT + nt * 32 + lc) * W6_STRIDE + 32 * sl + 16 * t + 8 * g);
      long xop[2][2];                            // [m tile][16-value group]
#pragma unroll
      for (int mt = 0; mt < 2; ++mt) {
        const uint8_t* ap = s.xa + (wm * 64 + mt * 32 + lc) * A6_STRIDE + 32 + 32 * sl + 8 * g;
        xop[mt][0] = *reinterpret_cast<const long*>(ap);
        xop[mt][1] = *reinterpret_cast<const long*>(ap + 16);
      }
      // Software pipeline over the 2 * NT (m tile, n tile) pairs: the two MFMAs of pair i+1 are issued before
      // the scale arithmetic of pair i.
      constexpr int PAIRS = 2 * NT;
      struct Dots { v16i d0, d1; };
      auto issue = [&](int i) {
        const int mt = i / NT, nt = i % NT;
        Dots r;
        r.d0 = __builtin_amdgcn_mfma_i32_32x32x16_i8(xop[mt][0], wop[nt][0], ci, 0, 0, 0);
        r.d1 = __builtin_amdgcn_mfma_i32_32x32x16_i8(xop[mt][1], wop[nt][1], ci, 0, 0, 0);
        return r;
      };
      Dots cur = issue(0);
#pragma unroll
      for (int i = 0; i < PAIRS; ++i) {
        const int mt = i / NT, nt = i % NT;
        Dots next = cur;
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
          for (int v = 0; v < 16; ++v) {
            const int row = wm * 64 + mt * 32 + 8 * (v >> 2) + 4 * g + (v & 3);
            dump(row, col, (step * 4 + sl) * 2, cur.d0[v] - static_cast<int>(MMQ_MAGIC_BITS));
            dump(row, col, (step * 4 + sl) * 2 + 1, cur.d1[v] - static_cast<int>(MMQ_MAGIC_BITS));
          }
        }
        const float s0 = s.sw[2 * sl][col], c0 = s.cw[2 * sl][col];
        const float s1 = s.sw[2 * sl + 1][col], c1 = s.cw[2 * sl + 1][col];
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const float t0 = __builtin_fmaf(bits_to_float(static_cast<uint32_t>(cur.d0[v])), s0, c0);   // s0 * dot0, rounded once
          const float t1 = __builtin_fmaf(bits_to_float(static_cast<uint32_t>(cur.d1[v])), s1, c1);
          acc[nt][mt][v] = __builtin_fmaf(xdv[v], t0 + t1, acc[nt][mt][v]);
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
