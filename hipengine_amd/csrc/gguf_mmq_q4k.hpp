// Tile engine of the Q4_K x DS4 MMQ GEMM on the gfx950 int8 MFMA, shared by the
// dense prefill GEMM and the expert-grouped (MoE) GEMM.
//
//   out[m,n] = sum_{32-wide sub-block j} (d*sc_j)[n] * xd_j[m] * dot_j[m,n] - (dmin*mn_j)[n] * xsum_j[m]
//   (kernels/hip_gfx1100/quant/gguf_q4_k_q8_1_mmq_prefill.hip:265-276)
//
// A workgroup of WM x WN waves computes a (32*MT*WM) x (32*NT*WN) output tile;
// each wave owns MT x NT MFMA tiles of 32x32.  One K step is 128 values: one
// DS4 activation block per row and half of a Q4_K block (two nibble pairs =
// four 32-wide sub-blocks) per column.
//   * The step's activation blocks and weight nibbles are copied to LDS with
//     16-byte loads; with PREFETCH the loads of step s+1 are issued into
//     registers before step s is computed.  A thread's byte offsets are
//     computed once per tile, a weight block's header is decoded once per
//     block, and the Q4_K format keeps two LDS copies of a step's images, so
//     the K loop has one barrier per step.
//   * A wave reads MFMA operands straight from those LDS images: the int8
//     activation bytes as they are, the weight nibbles split in registers.
//     v_mfma_i32_32x32x32_i8 spans exactly one sub-block, so every int32
//     result is an exact sub-block dot.
//   * The accumulator input of each MFMA is the integer 0x4B400000, so the
//     int32 result reinterpreted as float IS 12582912 + dot; one FMA with the
//     per-column constants (sw, -12582912*sw) yields the correctly rounded
//     sw*dot without an int->float conversion (12582912*sw is exact: sw = d*sc
//     has at most 17 significant bits), a second FMA applies the per-row
//     activation scale.
//   * The min term is rank-8 per Q4_K block: sum_j mn_j[n]*xsum_j[m] is one
//     v_mfma_f32_32x32x8f16 (both operands are exact in fp16: xsum is stored as
//     fp16, mn_j <= 63), scaled by dmin[n] once per block.
//
// The float32 epilogue (2 VALU ops per output element per sub-block, 64 lanes
// per CU-cycle) bounds this formulation at about a fifth of the int8 MFMA
// peak: the MFMA pipe itself is mostly idle.
#pragma once

#include <type_traits>

#include "gguf_common.hpp"

namespace hipengine_gfx950 {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr uint32_t MMQ_MAGIC_BITS = 0x4B400000u;   // float 12582912 = 1.5 * 2^23
constexpr float MMQ_MAGIC = 12582912.0f;

// FMT selects the operand formats of the same engine:
//   MMQ_Q4K_DS4   Q4_K weights x DS4 activations (fp16 scale and raw sum per 32 values, 144-byte blocks);
//   MMQ_Q5K_D4S4  Q5_K weights x D4S4 activations (float32 scale and raw sum per 32 values, 160-byte blocks):
//                 out = sum_j (d*sc_j)*xd_j*dot_j - (dmin*mn_j)*s4_j (gguf_k_mmq_prefill.hip:563-572,655-664).
//                 The fifth bit of a value comes from the block's qh bytes (bit s of qh[l] for sub-block s,
//                 value l), which travel to LDS beside the nibbles; the float32 raw sum enters the fp16 MFMA of
//                 the min term as a high and a low fp16 part (two MFMAs, the product with mn <= 63 exact).
enum MmqFormat : int { MMQ_Q4K_DS4 = 0, MMQ_Q5K_D4S4 = 1 };

template <int MT_, int NT_, int WM_, int WN_, int FMT = MMQ_Q4K_DS4>
struct Q4Tile {
  static constexpr int MT = MT_, NT = NT_, WM = WM_, WN = WN_;
  static constexpr bool Q5 = FMT == MMQ_Q5K_D4S4;
  static constexpr int BM = 32 * MT * WM, BN = 32 * NT * WN, THREADS = 64 * WM * WN;
  static constexpr int A_BYTES = Q5 ? D4S4_BYTES : DS4_BYTES;   // activation block
  static constexpr int A_PARTS = A_BYTES / 16;                  // 9 or 10 chunks of 16 bytes
  static constexpr int A_QS = Q5 ? 32 : 16;                     // offset of the 128 int8 values in the block
  static constexpr int A_STRIDE = Q5 ? 176 : DS4_BYTES;         // 9 or 11 x 16 B: conflict free for b128 reads
  static constexpr int W_BLOCK = Q5 ? Q5_K_BYTES : Q4_K_BYTES;
  static constexpr int W_QS = Q5 ? 48 : 16;                     // offset of the 128 nibble bytes in the block
  static constexpr int W_PARTS = Q5 ? 6 : 4;                    // 16-byte chunks per column and K step: 4 of nibbles (+ 2 of qh)
  static constexpr int W_STRIDE = Q5 ? 112 : 80;                // 64 nibble bytes (+ 32 qh bytes) per K step, padded to 5 / 7 x 16 B
  static constexpr int A_CHUNKS = BM * A_PARTS, W_CHUNKS = BN * W_PARTS, H_ITEMS = BN + BM;
  static constexpr int A_PER = (A_CHUNKS + THREADS - 1) / THREADS;
  static constexpr int W_PER = (W_CHUNKS + THREADS - 1) / THREADS;
  static constexpr int H_PER = (H_ITEMS + THREADS - 1) / THREADS;

  // Two copies of everything a K step stages, so a step's images are written while slower waves still read the
  // step before: one barrier per step.  What belongs to a step (values, nibbles, activation scales) alternates with
  // the step; what belongs to a weight block of two steps (scales, mins, activation sums) with the block.
  static constexpr int NBUF = Q5 ? 1 : 2;   // Q5_K x D4S4 images are too large to hold twice with two workgroups
                                            // on a CU: one copy, and a second barrier per step
  struct Smem {
    uint8_t xa[NBUF][BM * A_STRIDE];   // DS4 blocks of the step, as stored
    uint8_t wq[NBUF][BN * W_STRIDE];   // 64 nibble bytes per column
    float sw[NBUF][8][BN];             // d*sc of the eight sub-blocks of the weight block, by column (decoded at the
                                    // block's first K step, used by both)
    float xd[NBUF][4][BM];             // activation scale per sub-block of the step, by row
    float dmin[NBUF][BN];
    _Float16 mnh[NBUF][BN][8];         // 6-bit mins as fp16
    _Float16 xsh[NBUF][BM][8];         // activation sums of the weight block (fp16 in the DS4 block already; D4S4: high part)
    _Float16 xsl[NBUF][Q5 ? BM : 1][8];   // D4S4: low part of the float32 sums
  };

  // Registers of one K step in flight between global memory and LDS.
  struct Regs {
    u32x4 pa[A_PER];
    u32x4 pw[W_PER];
    u32x4 ph[H_PER];   // item < BN: weight block header of that column; else activation block header of row item-BN
    u32x4 ph2[Q5 ? H_PER : 1];   // D4S4: the second half of a row's header (the four float32 sums)
  };

  // What a thread fetches every K step, as byte offsets that do not change along K: from xq for its activation
  // chunks and row headers, from w for its nibble chunks and column headers.  The step adds a scalar to the base
  // (the loads then take a 64-bit scalar base and a 32-bit lane offset: no address arithmetic in the K loop).
  // Callers pass bases at the tile's first row and column, so 32 bits hold any offset within a tile; a caller
  // that gathers its rows from anywhere in a large buffer asks for 64-bit row offsets (WIDE).
  template <bool WIDE>
  struct Offsets {
    using Row = typename std::conditional<WIDE, uint64_t, uint32_t>::type;
    Row a[A_PER];
    uint32_t w[W_PER];
    Row h[H_PER];
  };

  template <bool WIDE, class RowOf, class ColOf>
  static __device__ __forceinline__ Offsets<WIDE> offsets(int64_t x_row_bytes, int64_t w_row_bytes, int tid, RowOf row_of,
                                                    ColOf col_of) {
    Offsets<WIDE> o;
    using Row = typename Offsets<WIDE>::Row;
#pragma unroll
    for (int i = 0; i < A_PER; ++i) {
      const int c = min(tid + i * THREADS, A_CHUNKS - 1);
      const int row = c / A_PARTS, part = c - row * A_PARTS;
      o.a[i] = static_cast<Row>(row_of(row) * x_row_bytes + part * 16);
    }
#pragma unroll
    for (int i = 0; i < W_PER; ++i) {
      const int c = min(tid + i * THREADS, W_CHUNKS - 1);
      const int col = c / W_PARTS, part = c - col * W_PARTS;
      // parts 0..3: the step's 64 nibble bytes (the step adds 64 h); Q5_K parts 4, 5: the block's 32 qh bytes
      o.w[i] = static_cast<uint32_t>(col_of(col) * w_row_bytes + (part < 4 ? W_QS + part * 16 : 16 + (part - 4) * 16));
    }
#pragma unroll
    for (int i = 0; i < H_PER; ++i) {
      const int item = min(tid + i * THREADS, H_ITEMS - 1);
      o.h[i] = static_cast<Row>(item < BN ? col_of(item) * w_row_bytes : row_of(item - BN) * x_row_bytes);
    }
    return o;
  }

  // `row_of(r)` / `col_of(c)` give the activation row (in DS4 blocks of x_row_bytes
  // per row from xq) and the weight row (of w_row_bytes from w) that tile row r /
  // tile column c read; rows and columns outside the problem are mapped to any
  // valid one by the caller (their results are not stored).
  template <bool WIDE>
  static __device__ __forceinline__ void load_w(const uint8_t* w, int step, int tid, const Offsets<WIDE>& o,
                                                u32x4 (&pw)[W_PER]) {
    const int kb = step >> 1, h = step & 1;
    const uint8_t* wb = w + static_cast<int64_t>(kb) * W_BLOCK;           // uniform
#pragma unroll
    for (int i = 0; i < W_PER; ++i) {
      if constexpr (Q5) {
        const int part = min(tid + i * THREADS, W_CHUNKS - 1) % W_PARTS;
        pw[i] = *reinterpret_cast<const u32x4*>(wb + o.w[i] + (part < 4 ? h * 64 : 0));
      } else {
        pw[i] = *reinterpret_cast<const u32x4*>(wb + h * 64 + o.w[i]);
      }
    }
  }

  // activation chunks and the headers of both sides
  template <bool WIDE>
  static __device__ __forceinline__ void load_ah(const uint8_t* xq, const uint8_t* w, int step, int tid,
                                                 const Offsets<WIDE>& o, Regs& r) {
    const int kb = step >> 1, h = step & 1;
    const uint8_t* xs = xq + static_cast<int64_t>(step) * A_BYTES;        // uniform
    const uint8_t* wb = w + static_cast<int64_t>(kb) * W_BLOCK;           // uniform
#pragma unroll
    for (int i = 0; i < A_PER; ++i) r.pa[i] = *reinterpret_cast<const u32x4*>(xs + o.a[i]);
#pragma unroll
    for (int i = 0; i < H_PER; ++i) {
      const int item = min(tid + i * THREADS, H_ITEMS - 1);
      if (item < BN) {
        if (h == 0) r.ph[i] = *reinterpret_cast<const u32x4*>(wb + o.h[i]);   // decoded once per block
      } else {
        r.ph[i] = *reinterpret_cast<const u32x4*>(xs + o.h[i]);
        if constexpr (Q5) r.ph2[i] = *reinterpret_cast<const u32x4*>(xs + o.h[i] + 16);
      }
    }
  }

  template <bool WIDE>
  static __device__ __forceinline__ void load(const uint8_t* xq, const uint8_t* w, int step, int tid,
                                              const Offsets<WIDE>& o, Regs& r) {
    load_w(w, step, tid, o, r.pw);
    load_ah(xq, w, step, tid, o, r);
  }

  static __device__ __forceinline__ void store(Smem& s, int step, int tid, const Regs& r, const u32x4 (&pw)[W_PER]) {
    const int h = step & 1, sb = step & (NBUF - 1), bb = (step >> 1) & (NBUF - 1);   // step half, step copy, block copy
#pragma unroll
    for (int i = 0; i < A_PER; ++i) {
      const int c = tid + i * THREADS;           // DS4: 144-byte rows are contiguous in LDS, offset c*16
      if (c < A_CHUNKS) {
        if constexpr (Q5) {
          const int row = c / A_PARTS, part = c - row * A_PARTS;
          *reinterpret_cast<u32x4*>(s.xa[sb] + row * A_STRIDE + part * 16) = r.pa[i];
        } else {
          *reinterpret_cast<u32x4*>(s.xa[sb] + c * 16) = r.pa[i];
        }
      }
    }
#pragma unroll
    for (int i = 0; i < W_PER; ++i) {
      const int c = tid + i * THREADS;
      if (c < W_CHUNKS) *reinterpret_cast<u32x4*>(s.wq[sb] + (c / W_PARTS) * W_STRIDE + (c % W_PARTS) * 16) = pw[i];
    }
#pragma unroll
    for (int i = 0; i < H_PER; ++i) {
      const int item = tid + i * THREADS;
      const u32x4 ph = r.ph[i];
      if (item < BN) {
        if (h == 0) {
          const Q4KScales u = q4k_unpack_scales(ph.y, ph.z, ph.w);
          const float d = f16_bits_to_float(ph.x & 0xFFFFu);
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const float sw = d * static_cast<float>(((j < 4 ? u.sc_lo : u.sc_hi) >> (8 * (j & 3))) & 0xFFu);
            s.sw[bb][j][item] = sw;
          }
          s.dmin[bb][item] = f16_bits_to_float(ph.x >> 16);
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const uint32_t mn = ((j < 4 ? u.mn_lo : u.mn_hi) >> (8 * (j & 3))) & 0xFFu;
            s.mnh[bb][item][j] = static_cast<_Float16>(static_cast<float>(mn));
          }
        }
      } else if (item < H_ITEMS) {
        const int row = item - BN;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          if constexpr (Q5) {
            s.xd[sb][j][row] = bits_to_float(ph[j]);
            const float sum = bits_to_float(r.ph2[i][j]);
            const _Float16 hi = static_cast<_Float16>(sum);
            s.xsh[bb][row][4 * h + j] = hi;
            s.xsl[bb][row][4 * h + j] = static_cast<_Float16>(sum - static_cast<float>(hi));
          } else {
            s.xd[sb][j][row] = f16_bits_to_float(ph[j] & 0xFFFFu);
            s.xsh[bb][row][4 * h + j] = __builtin_bit_cast(_Float16, static_cast<uint16_t>(ph[j] >> 16));
          }
        }
      }
    }
  }

  // One K step of MFMA work on the LDS images; acc is [NT][MT][16].  `dump(row, col, sub_block, dot)`
  // receives every int32 sub-block dot (tile-relative row and column, sub-block of the K step) when DUMP.
  template <bool DUMP = false, class Dump = int>
  static __device__ __forceinline__ void compute(const Smem& s, int step, int wm, int wn, int lc, int g,
                                                 float (&acc)[NT][MT][16], Dump dump = 0) {
    const int h = step & 1, sb = step & (NBUF - 1), bb = (step >> 1) & (NBUF - 1);
    v16i c0;
#pragma unroll
    for (int v = 0; v < 16; ++v) c0[v] = static_cast<int>(MMQ_MAGIC_BITS);
#pragma unroll
    for (int sp = 0; sp < 2; ++sp) {
      v4i wlo[NT], whi[NT];
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        const int col = (wn * NT + nt) * 32 + lc;
        const u32x4 qs = *reinterpret_cast<const u32x4*>(s.wq[sb] + col * W_STRIDE + sp * 32 + 16 * g);
        wlo[nt] = v4i{static_cast<int>(q4k_low(qs.x)), static_cast<int>(q4k_low(qs.y)),
                      static_cast<int>(q4k_low(qs.z)), static_cast<int>(q4k_low(qs.w))};
        whi[nt] = v4i{static_cast<int>(q4k_high(qs.x)), static_cast<int>(q4k_high(qs.y)),
                      static_cast<int>(q4k_high(qs.z)), static_cast<int>(q4k_high(qs.w))};
        if constexpr (Q5) {
          // values 16g..16g+15 of sub-blocks s0 = 4h + 2sp (low nibbles) and s0 + 1 (high): bit 4 is bit s of qh[l]
          const u32x4 qh = *reinterpret_cast<const u32x4*>(s.wq[sb] + col * W_STRIDE + 64 + 16 * g);
          const int s0 = 4 * h + 2 * sp;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            wlo[nt][e] |= static_cast<int>(((qh[e] >> s0) & 0x01010101u) << 4);
            whi[nt][e] |= static_cast<int>(((qh[e] >> (s0 + 1)) & 0x01010101u) << 4);
          }
        }
      }
      // The 2*MT*NT MFMAs of this nibble pair, software-pipelined: the MFMA of tile i+1 is issued
      // before the 32 scale FMAs of tile i, so the matrix pipe works while the VALU does.
      constexpr int TILES = 2 * MT * NT;          // tile i: half = i / (MT*NT), mt = (i / NT) % MT, nt = i % NT
      v4i xop[2][MT];
#pragma unroll
      for (int half = 0; half < 2; ++half)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          xop[half][mt] = *reinterpret_cast<const v4i*>(s.xa[sb] + ((wm * MT + mt) * 32 + lc) * A_STRIDE + A_QS +
                                                        (2 * sp + half) * 32 + 16 * g);
      auto issue = [&](int i) {
        const int half = i / (MT * NT), mt = (i / NT) % MT, nt = i % NT;
        return __builtin_amdgcn_mfma_i32_32x32x32_i8(xop[half][mt], half ? whi[nt] : wlo[nt], c0, 0, 0, 0);
      };
      // per (half, mt) pair: the activation scales of the lane's 16 rows and the column constants of its NT tiles
      // (reading them a pair ahead costs 20 registers and measured no faster)
      struct PairOps { float xdv[16]; float sw[NT], cw[NT]; };
      auto load_pair = [&](int pr) {
        const int half = pr / MT, mt = pr % MT;
        const int sl = 2 * sp + half;
        const int rbase = (wm * MT + mt) * 32;
        PairOps o;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float4 t = *reinterpret_cast<const float4*>(&s.xd[sb][sl][rbase + 8 * j + 4 * g]);
          o.xdv[4 * j] = t.x; o.xdv[4 * j + 1] = t.y; o.xdv[4 * j + 2] = t.z; o.xdv[4 * j + 3] = t.w;
        }
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
          const int col = (wn * NT + nt) * 32 + lc;
          o.sw[nt] = s.sw[bb][4 * h + sl][col]; o.cw[nt] = -MMQ_MAGIC * o.sw[nt];
        }
        return o;
      };
      v16i dcur = issue(0);
#pragma unroll
      for (int pr = 0; pr < 2 * MT; ++pr) {
        const int mt = pr % MT;
        const PairOps ops = load_pair(pr);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
          const int i = pr * NT + nt;
          v16i dnext = dcur;
          if (i + 1 < TILES) dnext = issue(i + 1);
          if constexpr (DUMP) {
#pragma unroll
            for (int v = 0; v < 16; ++v)
              dump((wm * MT + mt) * 32 + 8 * (v >> 2) + 4 * g + (v & 3), (wn * NT + nt) * 32 + lc, 2 * sp + pr / MT,
                   dcur[v] - static_cast<int>(MMQ_MAGIC_BITS));
          }
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const float t = __builtin_fmaf(bits_to_float(static_cast<uint32_t>(dcur[v])), ops.sw[nt], ops.cw[nt]);   // = sw * dot, rounded once
            acc[nt][mt][v] = __builtin_fmaf(ops.xdv[v], t, acc[nt][mt][v]);
          }
          dcur = dnext;
        }
      }
    }

    // min term, once per Q4_K block: dmin[n] * sum_j mn_j[n] * xsum_j[m] on the fp16 MFMA
    if (h == 1) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const int arow = (wm * MT + mt) * 32 + lc;
        const v4h xs = *reinterpret_cast<const v4h*>(&s.xsh[bb][arow][4 * g]);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
          const int col = (wn * NT + nt) * 32 + lc;
          const v4h mn = *reinterpret_cast<const v4h*>(&s.mnh[bb][col][4 * g]);
          v16f z;
#pragma unroll
          for (int v = 0; v < 16; ++v) z[v] = 0.0f;
          v16f t = __builtin_amdgcn_mfma_f32_32x32x8f16(xs, mn, z, 0, 0, 0);
          if constexpr (Q5) {
            const v4h xl = *reinterpret_cast<const v4h*>(&s.xsl[bb][arow][4 * g]);
            t = __builtin_amdgcn_mfma_f32_32x32x8f16(xl, mn, t, 0, 0, 0);
          }
          const float nd = -s.dmin[bb][col];
#pragma unroll
          for (int v = 0; v < 16; ++v) acc[nt][mt][v] = __builtin_fmaf(nd, t[v], acc[nt][mt][v]);
        }
      }
    }
  }

  // The whole K loop of one output tile.  `emit(row, col, value)` receives every
  // element of the tile (tile-relative coordinates) once.
  template <bool PREFETCH, bool WIDE_ROWS, class RowOf, class ColOf, class Emit, bool DUMP = false, class Dump = int>
  static __device__ __forceinline__ void run(const uint8_t* xq, int64_t x_row_bytes, const uint8_t* w,
                                             int64_t w_row_bytes, int steps, Smem& s, RowOf row_of, ColOf col_of,
                                             Emit emit, Dump dump = 0) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave % WM, wn = wave / WM;
    const int lc = lane & 31, g = lane >> 5;

    float acc[NT][MT][16];
#pragma unroll
    for (int i = 0; i < NT; ++i)
#pragma unroll
      for (int j = 0; j < MT; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    const Offsets<WIDE_ROWS> offs = offsets<WIDE_ROWS>(x_row_bytes, w_row_bytes, tid, row_of, col_of);
    Regs regs;
    auto work = [&](int step) {
      if constexpr (DUMP) {
        compute<true>(s, step, wm, wn, lc, g, acc, [&](int row, int col, int sb, int dot) { dump(row, col, 4 * step + sb, dot); });
      } else {
        compute(s, step, wm, wn, lc, g, acc);
      }
    };
    if (PREFETCH) load(xq, w, 0, tid, offs, regs);
    for (int step = 0; step < steps; ++step) {
      if (!PREFETCH) load(xq, w, step, tid, offs, regs);
      store(s, step, tid, regs, regs.pw);
      __syncthreads();
      // The loads of the next step are issued before this step is computed, so
      // their latency hides behind the MFMA/FMA work.
      if (PREFETCH && step + 1 < steps) load(xq, w, step + 1, tid, offs, regs);
      work(step);
      // two copies: no barrier here.  The next step writes the other copy, and whoever writes this copy again
      // (two steps on) has passed the next step's barrier, which every wave reaches only after this compute
      if constexpr (NBUF == 1) __syncthreads();
    }

    // lane holds column lc of each n tile and rows 8*(v/4) + 4*g + v%4 of each m tile
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int v = 0; v < 16; ++v)
          emit((wm * MT + mt) * 32 + 8 * (v >> 2) + 4 * g + (v & 3), (wn * NT + nt) * 32 + lc, acc[nt][mt][v]);
  }
};

}  // namespace hipengine_gfx950
