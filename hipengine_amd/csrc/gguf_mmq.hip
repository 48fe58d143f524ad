// MMQ prefill GEMM on int8 MFMA for gfx950: raw Q4_K weights x DS4 q8_1
// activations -> float32 / bf16, and raw Q6_K weights x D4S4 activations.
//
//   Q4_K: out[m,n] = sum_{32-wide sub-block j} (d*sc_j)[n] * xd_j[m] * dot_j[m,n] - (dmin*mn_j)[n] * xsum_j[m]
//         (kernels/hip_gfx1100/quant/gguf_q4_k_q8_1_mmq_prefill.hip:265-276)
//   Q6_K: out[m,n] = sum_{32-wide group g} xd_g[m] * (s0*dot0 + s1*dot1),  s = d*scale_i8, dots over 16 values
//         (kernels/hip_gfx1100/quant/gguf_k_mmq_prefill.hip:652-667)
//
// Both run 256 threads = 4 waves on a 128x128 output tile, each wave 64x64 as
// 2x2 MFMA tiles of 32x32, one 128-value K step at a time.  The Q4_K tile
// engine is in gguf_mmq_q4k.hpp; the Q6_K kernel below follows the same plan
// with v_mfma_i32_32x32x16_i8 per 16 values.

#include "gguf_mmq_q4k.hpp"

#include "gguf_init.hpp"

#include "../../include/hipengine_gfx950.h"
#include "../../include/hipengine_gfx950_tuning.h"

namespace {

using namespace hipengine_gfx950;

using DenseQ4 = Q4Tile<2, 2, 2, 2>;
constexpr int BM = DenseQ4::BM, BN = DenseQ4::BN, THREADS = DenseQ4::THREADS;
constexpr uint32_t MAGIC_BITS = MMQ_MAGIC_BITS;
constexpr float MAGIC = MMQ_MAGIC;

struct MmqArgs {
  const uint8_t* xq;
  const uint8_t* w;
  void* out;
  int out_kind;
  int M, K, N;
};

__device__ __forceinline__ void store_tile(const MmqArgs& a, const float (&acc)[16], int m_base, int n_col) {
  // lane holds column n_col and rows m_base + 8*(v/4) + v%4 (m_base already includes 4*(lane/32))
  if (n_col >= a.N) return;
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int m = m_base + 8 * (v >> 2) + (v & 3);
    if (m < a.M) store_scalar(a.out, static_cast<int64_t>(m) * a.N + n_col, acc[v], a.out_kind);
  }
}

// Tiles of 32x64 or 64x32 per wave on 8 waves (half the accumulators, 3 or 4 waves per SIMD instead of 2) spill
// registers in the K loop and measured 450-480 int8 TOPS against 668 for 64x64 per wave on 4 waves (M = 2048,
// 17408x5120).
template <class Tile, bool PREFETCH, int MIN_WAVES>
__global__ void __launch_bounds__(Tile::THREADS, MIN_WAVES) mmq_q4_k_ds4_kernel(MmqArgs a) {
  extern __shared__ __align__(16) uint8_t smem_raw[];
  typename Tile::Smem& s = *reinterpret_cast<typename Tile::Smem*>(smem_raw);
  const int m0 = blockIdx.x * Tile::BM, n0 = blockIdx.y * Tile::BN;
  const int steps = a.K / 128;
  const int64_t w_row_bytes = static_cast<int64_t>(a.K / QK_K) * Tile::W_BLOCK;
  const int64_t x_row_bytes = static_cast<int64_t>(steps) * Tile::A_BYTES;
  Tile::template run<PREFETCH>(
      a.xq, x_row_bytes, a.w, w_row_bytes, steps, s,
      [=](int row) { return static_cast<int64_t>(min(m0 + row, a.M - 1)); },
      [=](int col) { return static_cast<int64_t>(min(n0 + col, a.N - 1)); },
      [=](int row, int col, float v) {
        const int m = m0 + row, n = n0 + col;
        if (m < a.M && n < a.N) store_scalar(a.out, static_cast<int64_t>(m) * a.N + n, v, a.out_kind);
      });
}

template <class Tile, bool PREFETCH, int MIN_WAVES>
void launch_q4_tile(const MmqArgs& a, hipStream_t stream) {
  const dim3 grid(static_cast<unsigned>((a.M + Tile::BM - 1) / Tile::BM), static_cast<unsigned>((a.N + Tile::BN - 1) / Tile::BN));
  hipLaunchKernelGGL((mmq_q4_k_ds4_kernel<Tile, PREFETCH, MIN_WAVES>), grid, dim3(Tile::THREADS), sizeof(typename Tile::Smem),
                     stream, a);
}

// Verification: the same tile engine, which also writes every int32 sub-block dot to dots[M, N, K/32].
template <class Tile>
__global__ void __launch_bounds__(Tile::THREADS, 2) mmq_tile_dump_kernel(MmqArgs a, int32_t* __restrict__ dots) {
  extern __shared__ __align__(16) uint8_t smem_raw[];
  typename Tile::Smem& s = *reinterpret_cast<typename Tile::Smem*>(smem_raw);
  const int m0 = blockIdx.x * Tile::BM, n0 = blockIdx.y * Tile::BN;
  const int steps = a.K / 128;
  const int64_t w_row_bytes = static_cast<int64_t>(a.K / QK_K) * Tile::W_BLOCK;
  const int64_t x_row_bytes = static_cast<int64_t>(steps) * Tile::A_BYTES;
  auto row_of = [=](int row) { return static_cast<int64_t>(min(m0 + row, a.M - 1)); };
  auto col_of = [=](int col) { return static_cast<int64_t>(min(n0 + col, a.N - 1)); };
  auto emit = [=](int row, int col, float v) {
    const int m = m0 + row, n = n0 + col;
    if (m < a.M && n < a.N) store_scalar(a.out, static_cast<int64_t>(m) * a.N + n, v, a.out_kind);
  };
  auto dump = [=](int row, int col, int sb, int dot) {
    const int m = m0 + row, n = n0 + col;
    if (m < a.M && n < a.N) dots[(static_cast<int64_t>(m) * a.N + n) * (a.K / 32) + sb] = dot;
  };
  Tile::template run<true, decltype(row_of), decltype(col_of), decltype(emit), true, decltype(dump)>(
      a.xq, x_row_bytes, a.w, w_row_bytes, steps, s, row_of, col_of, emit, dump);
}

int launch_q4(const void* xq, const uint8_t* w, void* out, int out_kind, int64_t M, int64_t K, int64_t N,
              int variant, hipStream_t stream) {
  if (!xq || !w || !out || M <= 0 || M > (1 << 20) || K <= 0 || (K % QK_K) != 0 || N <= 0 || (N % 32) != 0 ||
      N > (1 << 24) || out_kind < KIND_F32 || out_kind > KIND_F16) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  MmqArgs a{static_cast<const uint8_t*>(xq), w, out, out_kind, static_cast<int>(M), static_cast<int>(K),
            static_cast<int>(N)};
  switch (variant) {
    case 1: launch_q4_tile<DenseQ4, false, 2>(a, stream); break;
    default: launch_q4_tile<DenseQ4, true, 2>(a, stream); break;
  }
  return static_cast<int>(hipGetLastError());
}

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
  uint8_t xa[BM * A6_STRIDE];
  uint8_t w8[COLS * W6_STRIDE];
  float sw[8][COLS];   // d * scale of the 8 16-value groups of the step, by column
  float cw[8][COLS];   // -MAGIC * sw (exact: d has 11 significant bits, the scale 8)
  float xd[4][BM];     // activation scale per 32 values, by row
};

struct Q6StepRegs {
  u32x4 pa[5];         // 128 rows x 10 chunks = 1280 = 5 per thread
  u32x4 qla, qlb, qh;  // 16 bytes each of the column tid/2, byte offset 16*(tid&1)
  uint2 sc;            // threads 0..COLS-1: the 8 scales of column tid
  uint32_t d;          //                    and its fp16 d
  u32x4 xd;            // threads COLS..COLS+127: the four float scales of row tid-COLS
};

template <int COLS>
__device__ __forceinline__ void q6_step_load(const MmqArgs& a, int step, int m0, int n0, int64_t w_row_bytes,
                                             int64_t x_row_bytes, int tid, Q6StepRegs& r) {
  const int kb = step >> 1, hh = step & 1;
#pragma unroll
  for (int i = 0; i < 5; ++i) {
    const int c = tid + i * THREADS;
    const int row = c / 10, part = c - row * 10;
    const int m = min(m0 + row, a.M - 1);
    r.pa[i] = *reinterpret_cast<const u32x4*>(a.xq + m * x_row_bytes + static_cast<int64_t>(step) * D4S4_BYTES + part * 16);
  }
  if (tid < 2 * COLS) {
    const int n = min(n0 + (tid >> 1), a.N - 1);
    const uint8_t* blk = a.w + n * w_row_bytes + static_cast<int64_t>(kb) * Q6_K_BYTES;
    const int o = (tid & 1) * 16;
    const uint4 x = load16(blk + 64 * hh + o), y = load16(blk + 64 * hh + 32 + o), z = load16(blk + 128 + 32 * hh + o);
    r.qla = u32x4{x.x, x.y, x.z, x.w};
    r.qlb = u32x4{y.x, y.y, y.z, y.w};
    r.qh = u32x4{z.x, z.y, z.z, z.w};
  }
  if (tid < COLS) {
    const uint8_t* blk = a.w + min(n0 + tid, a.N - 1) * w_row_bytes + static_cast<int64_t>(kb) * Q6_K_BYTES;
    r.sc = load8(blk + 192 + 8 * hh);
    r.d = load2(blk + 208);
  } else if (tid < COLS + BM) {
    r.xd = *reinterpret_cast<const u32x4*>(a.xq + min(m0 + tid - COLS, a.M - 1) * x_row_bytes +
                                           static_cast<int64_t>(step) * D4S4_BYTES);
  }
}

template <int COLS>
__device__ __forceinline__ void q6_step_store(Q6Smem<COLS>& s, int tid, const Q6StepRegs& r) {
#pragma unroll
  for (int i = 0; i < 5; ++i) {
    const int c = tid + i * THREADS;
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
      s.cw[j][tid] = -MAGIC * sw;
    }
  } else if (tid < COLS + BM) {
#pragma unroll
    for (int j = 0; j < 4; ++j) s.xd[j][tid - COLS] = bits_to_float(r.xd[j]);
  }
}

// DUMP: the verification instantiation, which also writes every int32 16-value dot to dots[M, N, K/16].
template <bool DUMP, int COLS = BN>
__global__ void __launch_bounds__(THREADS, 2) mmq_q6_k_d4s4_kernel(MmqArgs a, int32_t* __restrict__ dots) {
  static_assert(COLS == 128 || COLS == 64, "two wave columns of one or two 32-wide tiles");
  constexpr int NT = COLS / 64;                   // 32-wide n tiles per wave
  extern __shared__ __align__(16) uint8_t smem_raw[];
  Q6Smem<COLS>& s = *reinterpret_cast<Q6Smem<COLS>*>(smem_raw);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave & 1, wn = wave >> 1;
  const int lc = lane & 31, g = lane >> 5;
  const int m0 = blockIdx.x * BM, n0 = blockIdx.y * COLS;
  const int steps = a.K / 128;
  const int64_t w_row_bytes = static_cast<int64_t>(a.K / QK_K) * Q6_K_BYTES;
  const int64_t x_row_bytes = static_cast<int64_t>(steps) * D4S4_BYTES;

  float acc[NT][2][16];
#pragma unroll
  for (int i = 0; i < NT; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  Q6StepRegs regs;
  q6_step_load<COLS>(a, 0, m0, n0, w_row_bytes, x_row_bytes, tid, regs);

  for (int step = 0; step < steps; ++step) {
    q6_step_store(s, tid, regs);
    __syncthreads();
    if (step + 1 < steps) q6_step_load<COLS>(a, step + 1, m0, n0, w_row_bytes, x_row_bytes, tid, regs);

    v16i ci;
#pragma unroll
    for (int v = 0; v < 16; ++v) ci[v] = static_cast<int>(MAGIC_BITS);
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
            const int m = m0 + wm * 64 + mt * 32 + 8 * (v >> 2) + 4 * g + (v & 3), nn = n0 + col;
            if (m < a.M && nn < a.N) {
              int32_t* o = dots + (static_cast<int64_t>(m) * a.N + nn) * (a.K / 16) + (step * 4 + sl) * 2;
              o[0] = cur.d0[v] - static_cast<int>(MAGIC_BITS);
              o[1] = cur.d1[v] - static_cast<int>(MAGIC_BITS);
            }
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

#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
      store_tile(a, acc[nt][mt], m0 + wm * 64 + mt * 32 + 4 * g, n0 + wn * 32 * NT + nt * 32 + lc);
}

#ifndef Q6_TILE_CHOICE
#define Q6_TILE_CHOICE(wide_fill, narrow_fill) ((wide_fill) < 0.7 && (narrow_fill) > (wide_fill) + 0.1)
#endif
int launch_q6(const void* xq, const uint8_t* w, void* out, int out_kind, int64_t M, int64_t K, int64_t N,
              hipStream_t stream) {
  if (!xq || !w || !out || M <= 0 || M > (1 << 20) || K <= 0 || (K % QK_K) != 0 || N <= 0 || N > (1 << 24) ||
      out_kind < KIND_F32 || out_kind > KIND_F16) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  MmqArgs a{static_cast<const uint8_t*>(xq), w, out, out_kind, static_cast<int>(M), static_cast<int>(K),
            static_cast<int>(N)};
  // 128-wide tiles unless their last round of the 512 resident workgroups would be less than half full and
  // 64-wide tiles fill their rounds better (N = 5120 at M = 2048: 640 tiles = 1.25 rounds against 1280 = 2.5)
  const int64_t m_tiles = (M + BM - 1) / BM;
  const int64_t wide = m_tiles * ((N + 127) / 128), narrow = m_tiles * ((N + 63) / 64);
  const int64_t slots = 2 * 256;
  auto fill = [&](int64_t tiles) { return static_cast<double>(tiles) / static_cast<double>((tiles + slots - 1) / slots * slots); };
  if (Q6_TILE_CHOICE(fill(wide), fill(narrow))) {
    const dim3 grid(static_cast<unsigned>(m_tiles), static_cast<unsigned>((N + 63) / 64));
    hipLaunchKernelGGL((mmq_q6_k_d4s4_kernel<false, 64>), grid, dim3(THREADS), sizeof(Q6Smem<64>), stream, a,
                       static_cast<int32_t*>(nullptr));
  } else {
    const dim3 grid(static_cast<unsigned>(m_tiles), static_cast<unsigned>((N + BN - 1) / BN));
    hipLaunchKernelGGL((mmq_q6_k_d4s4_kernel<false, 128>), grid, dim3(THREADS), sizeof(Q6Smem<128>), stream, a,
                       static_cast<int32_t*>(nullptr));
  }
  return static_cast<int>(hipGetLastError());
}

}  // namespace

extern "C" int hipengine_gfx950_gguf_q4_k_mmq_tuned(const void* xq, const uint8_t* qweight, void* out, int out_kind,
                                                   int64_t rows, int64_t in_features, int64_t out_features,
                                                   int variant, hipStream_t stream) {
  return launch_q4(xq, qweight, out, out_kind, rows, in_features, out_features, variant, stream);
}

#define DEFINE_MMQ_Q4(SYMBOL, OKIND)                                                                        \
  extern "C" int SYMBOL(const void* xq, const uint8_t* qweight, void* out, int64_t rows, int64_t in_features, \
                        int64_t out_features, hipStream_t stream) {                                         \
    return launch_q4(xq, qweight, out, OKIND, rows, in_features, out_features, 0, stream);                     \
  }

DEFINE_MMQ_Q4(hipengine_gguf_q4_k_q8_1_mmq32_vdr_dense_bf16_f32_out, KIND_F32)
DEFINE_MMQ_Q4(hipengine_gguf_q4_k_q8_1_mmq32_vdr_dense_bf16_bf16_out, KIND_BF16)
DEFINE_MMQ_Q4(hipengine_gguf_q4_k_q8_1_mmq32_ctl_dense_bf16_f32_out, KIND_F32)
DEFINE_MMQ_Q4(hipengine_gguf_q4_k_q8_1_mmq32_ctl_dense_bf16_bf16_out, KIND_BF16)

// Q5_K x D4S4: the same tile engine with the fifth bit and float32 activation scales and sums.
using DenseQ5 = Q4Tile<2, 2, 2, 2, MMQ_Q5K_D4S4>;

int launch_q5(const void* xq, const uint8_t* w, void* out, int out_kind, int64_t M, int64_t K, int64_t N,
              hipStream_t stream) {
  if (!xq || !w || !out || M <= 0 || M > (1 << 20) || K <= 0 || (K % QK_K) != 0 || N <= 0 || (N % 32) != 0 ||
      N > (1 << 24) || out_kind < KIND_F32 || out_kind > KIND_F16) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  MmqArgs a{static_cast<const uint8_t*>(xq), w, out, out_kind, static_cast<int>(M), static_cast<int>(K),
            static_cast<int>(N)};
  // without the register prefetch of the next step: with it this format spills 20 registers in the K loop
  // (752 us against 666 at M = 2048, 17408x5120)
  launch_q4_tile<DenseQ5, false, 2>(a, stream);
  return static_cast<int>(hipGetLastError());
}

#define DEFINE_MMQ_Q5(SYMBOL, OKIND)                                                                        \
  extern "C" int SYMBOL(const void* xq, const uint8_t* qweight, void* out, int64_t rows, int64_t in_features, \
                        int64_t out_features, hipStream_t stream) {                                         \
    return launch_q5(xq, qweight, out, OKIND, rows, in_features, out_features, stream);                     \
  }

DEFINE_MMQ_Q5(hipengine_gguf_q5_k_mmq32_q8_1_d4s4_f32_bf16_f32_out, KIND_F32)
DEFINE_MMQ_Q5(hipengine_gguf_q5_k_mmq32_q8_1_d4s4_f32_bf16_bf16_out, KIND_BF16)

#define DEFINE_MMQ_Q6(SYMBOL, OKIND)                                                                        \
  extern "C" int SYMBOL(const void* xq, const uint8_t* qweight, void* out, int64_t rows, int64_t in_features, \
                        int64_t out_features, hipStream_t stream) {                                         \
    return launch_q6(xq, qweight, out, OKIND, rows, in_features, out_features, stream);                     \
  }

DEFINE_MMQ_Q6(hipengine_gguf_q6_k_mmq32_q8_1_d4s4_f32_bf16_f32_out, KIND_F32)
DEFINE_MMQ_Q6(hipengine_gguf_q6_k_mmq32_q8_1_d4s4_f32_bf16_bf16_out, KIND_BF16)

// ---- verification: the int32 dots the MMQ kernels feed their float32 combine with ----

extern "C" int hipengine_gfx950_gguf_mmq_dots_i32(int32_t ggml_type, const void* xq, const uint8_t* qweight,
                                                  int32_t* dots, float* out, int64_t rows, int64_t in_features,
                                                  int64_t out_features, hipStream_t stream) {
  if (!xq || !qweight || !dots || !out || rows <= 0 || rows > (1 << 20) || in_features <= 0 ||
      (in_features % QK_K) != 0 || out_features <= 0 || out_features > (1 << 24)) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  MmqArgs a{static_cast<const uint8_t*>(xq), qweight, out, KIND_F32, static_cast<int>(rows),
            static_cast<int>(in_features), static_cast<int>(out_features)};
  const dim3 grid(static_cast<unsigned>((rows + BM - 1) / BM), static_cast<unsigned>((out_features + BN - 1) / BN));
  if (ggml_type == GGML_Q4_K) {
    if ((out_features % 32) != 0) return static_cast<int>(hipErrorInvalidValue);
    hipLaunchKernelGGL(mmq_tile_dump_kernel<DenseQ4>, grid, dim3(THREADS), sizeof(DenseQ4::Smem), stream, a, dots);
  } else if (ggml_type == GGML_Q5_K) {
    if ((out_features % 32) != 0) return static_cast<int>(hipErrorInvalidValue);
    hipLaunchKernelGGL(mmq_tile_dump_kernel<DenseQ5>, grid, dim3(THREADS), sizeof(DenseQ5::Smem), stream, a, dots);
  } else if (ggml_type == GGML_Q6_K) {
    hipLaunchKernelGGL((mmq_q6_k_d4s4_kernel<true, 128>), grid, dim3(THREADS), sizeof(Q6Smem<128>), stream, a, dots);
  } else {
    return static_cast<int>(hipErrorInvalidValue);
  }
  return static_cast<int>(hipGetLastError());
}

// ---- prefill from bf16 activations: pack into the caller's workspace, then the MMQ ----

extern "C" int hipengine_gfx950_gguf_prefill_workspace_bytes(int32_t ggml_type, int64_t rows, int64_t in_features,
                                                             int64_t* bytes) {
  if (!bytes || rows <= 0 || in_features <= 0 || (in_features % QK_K) != 0 ||
      (ggml_type != GGML_Q4_K && ggml_type != GGML_Q5_K && ggml_type != GGML_Q6_K)) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  *bytes = rows * (in_features / 128) * (ggml_type == GGML_Q4_K ? DS4_BYTES : D4S4_BYTES);
  return static_cast<int>(hipSuccess);
}

extern "C" int hipengine_gfx950_gguf_prefill_bf16(int32_t ggml_type, const void* x, const uint8_t* qweight, void* out,
                                                  int32_t out_kind, int64_t rows, int64_t in_features,
                                                  int64_t out_features, void* workspace, int64_t workspace_bytes,
                                                  hipStream_t stream) {
  int64_t need = 0;
  const int rc = hipengine_gfx950_gguf_prefill_workspace_bytes(ggml_type, rows, in_features, &need);
  if (rc != static_cast<int>(hipSuccess)) return rc;
  if (!x || !workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 15u) != 0) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  if (ggml_type == GGML_Q4_K) {
    if ((out_features % 32) != 0) return static_cast<int>(hipErrorInvalidValue);
    const int prc = hipengine_gguf_q8_1_mmq_ds4_pack_bf16(x, workspace, rows, in_features, stream);
    if (prc != static_cast<int>(hipSuccess)) return prc;
    return launch_q4(workspace, qweight, out, out_kind, rows, in_features, out_features, 0, stream);
  }
  const int prc = hipengine_gguf_q8_1_d4s4_f32_quantize_bf16(x, workspace, rows, in_features, stream);
  if (prc != static_cast<int>(hipSuccess)) return prc;
  if (ggml_type == GGML_Q5_K) {
    if ((out_features % 32) != 0) return static_cast<int>(hipErrorInvalidValue);
    return launch_q5(workspace, qweight, out, out_kind, rows, in_features, out_features, stream);
  }
  return launch_q6(workspace, qweight, out, out_kind, rows, in_features, out_features, stream);
}

int hipengine_gfx950::mmq_load() {
  hipFuncAttributes attr;
  return static_cast<int>(hipFuncGetAttributes(&attr, reinterpret_cast<const void*>(mmq_q6_k_d4s4_kernel<false, 128>)));
}
