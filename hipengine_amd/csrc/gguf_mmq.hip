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
// engine is in gguf_mmq_q4k.hpp; the Q6_K engine (gguf_mmq_q6k.hpp) follows the same plan
// with v_mfma_i32_32x32x16_i8 per 16 values.

#include "gguf_mmq_q4k.hpp"
#include "gguf_mmq_q6k.hpp"
#include "gguf_mmq_q8_0.hpp"

#include "gguf_init.hpp"

#include <atomic>

#include "../../include/hipengine_gfx950.h"
#include "../../include/hipengine_gfx950_tuning.h"

namespace {

using namespace hipengine_gfx950;

using DenseQ4 = Q4Tile<2, 2, 2, 2>;
constexpr int BM = DenseQ4::BM, BN = DenseQ4::BN, THREADS = DenseQ4::THREADS;

struct MmqArgs {
  const uint8_t* xq;
  const uint8_t* w;
  void* out;
  int out_kind;
  int M, K, N;
};

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
  // rows and columns relative to the tile's first: the engine keeps 32-bit byte offsets from the two bases
  Tile::template run<PREFETCH, false>(
      a.xq + m0 * x_row_bytes, x_row_bytes, a.w + n0 * w_row_bytes, w_row_bytes, steps, s,
      [=](int row) { return static_cast<int64_t>(min(row, a.M - 1 - m0)); },
      [=](int col) { return static_cast<int64_t>(min(col, a.N - 1 - n0)); },
      [=](int row, int col, float v) {
        const int m = m0 + row, n = n0 + col;
        if (m < a.M && n < a.N) store_scalar(a.out, static_cast<int64_t>(m) * a.N + n, v, a.out_kind);
      });
}

template <class Tile, bool PREFETCH, int MIN_WAVES>
int launch_q4_tile(const MmqArgs& a, hipStream_t stream) {
  if (sizeof(typename Tile::Smem) > 65536) {   // the LDS limit is raised at set-up
    const int rc = ensure_init();
    if (rc != static_cast<int>(hipSuccess)) return rc;
  }
  const dim3 grid(static_cast<unsigned>((a.M + Tile::BM - 1) / Tile::BM), static_cast<unsigned>((a.N + Tile::BN - 1) / Tile::BN));
  hipLaunchKernelGGL((mmq_q4_k_ds4_kernel<Tile, PREFETCH, MIN_WAVES>), grid, dim3(Tile::THREADS), sizeof(typename Tile::Smem),
                     stream, a);
  return static_cast<int>(hipGetLastError());
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
  auto row_of = [=](int row) { return static_cast<int64_t>(min(row, a.M - 1 - m0)); };
  auto col_of = [=](int col) { return static_cast<int64_t>(min(col, a.N - 1 - n0)); };
  auto emit = [=](int row, int col, float v) {
    const int m = m0 + row, n = n0 + col;
    if (m < a.M && n < a.N) store_scalar(a.out, static_cast<int64_t>(m) * a.N + n, v, a.out_kind);
  };
  auto dump = [=](int row, int col, int sb, int dot) {
    const int m = m0 + row, n = n0 + col;
    if (m < a.M && n < a.N) dots[(static_cast<int64_t>(m) * a.N + n) * (a.K / 32) + sb] = dot;
  };
  Tile::template run<true, false, decltype(row_of), decltype(col_of), decltype(emit), true, decltype(dump)>(
      a.xq + m0 * x_row_bytes, x_row_bytes, a.w + n0 * w_row_bytes, w_row_bytes, steps, s, row_of, col_of, emit, dump);
}

int launch_q4(const void* xq, const uint8_t* w, void* out, int out_kind, int64_t M, int64_t K, int64_t N,
              int variant, hipStream_t stream) {
  if (!xq || !w || !out || M <= 0 || M > (1 << 20) || K <= 0 || (K % QK_K) != 0 || N <= 0 || (N % 32) != 0 ||
      N > (1 << 24) || out_kind < KIND_F32 || out_kind > KIND_F16) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  MmqArgs a{static_cast<const uint8_t*>(xq), w, out, out_kind, static_cast<int>(M), static_cast<int>(K),
            static_cast<int>(N)};
  return variant == 1 ? launch_q4_tile<DenseQ4, false, 2>(a, stream) : launch_q4_tile<DenseQ4, true, 2>(a, stream);
}

// --------------------------------------------------------------------------
// Q6_K x D4S4: the tile engine of gguf_mmq_q6k.hpp over the dense problem.
// DUMP: the verification instantiation, which also writes every int32 16-value dot to dots[M, N, K/16].
// --------------------------------------------------------------------------
template <bool DUMP, int COLS = BN>
__global__ void __launch_bounds__(THREADS, 2) mmq_q6_k_d4s4_kernel(MmqArgs a, int32_t* __restrict__ dots) {
  extern __shared__ __align__(16) uint8_t smem_raw[];
  Q6Smem<COLS>& s = *reinterpret_cast<Q6Smem<COLS>*>(smem_raw);
  const int m0 = blockIdx.x * BM, n0 = blockIdx.y * COLS;
  const int steps = a.K / 128;
  const int64_t w_row_bytes = static_cast<int64_t>(a.K / QK_K) * Q6_K_BYTES;
  const int64_t x_row_bytes = static_cast<int64_t>(steps) * D4S4_BYTES;
  auto row_of = [=](int row) { return static_cast<int64_t>(min(m0 + row, a.M - 1)); };
  auto col_of = [=](int col) { return static_cast<int64_t>(min(n0 + col, a.N - 1)); };
  auto emit = [=](int row, int col, float v) {
    const int m = m0 + row, n = n0 + col;
    if (m < a.M && n < a.N) store_scalar(a.out, static_cast<int64_t>(m) * a.N + n, v, a.out_kind);
  };
  if constexpr (DUMP) {
    q6_tile_run<true, COLS>(a.xq, x_row_bytes, a.w, w_row_bytes, steps, s, row_of, col_of, emit,
                            [=](int row, int col, int group, int dot) {
                              const int m = m0 + row, n = n0 + col;
                              if (m < a.M && n < a.N) dots[(static_cast<int64_t>(m) * a.N + n) * (a.K / 16) + group] = dot;
                            });
  } else {
    q6_tile_run<false, COLS>(a.xq, x_row_bytes, a.w, w_row_bytes, steps, s, row_of, col_of, emit);
  }
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

// --------------------------------------------------------------------------
// Q8_0 x D4S4: the tile engine of gguf_mmq_q8_0.hpp over the dense problem.
// DUMP: the verification instantiation, which also writes every int32 block dot to dots[M, N, K/32].
// --------------------------------------------------------------------------
template <bool DUMP, int COLS = BN>
__global__ void __launch_bounds__(THREADS, 2) mmq_q8_0_d4s4_kernel(MmqArgs a, int32_t* __restrict__ dots) {
  extern __shared__ __align__(16) uint8_t smem_raw[];
  Q8Smem<COLS>& s = *reinterpret_cast<Q8Smem<COLS>*>(smem_raw);
  const int m0 = blockIdx.x * BM, n0 = blockIdx.y * COLS;
  const int steps = a.K / 128;
  const int64_t w_row_bytes = static_cast<int64_t>(a.K / 32) * Q8_0_BYTES;
  const int64_t x_row_bytes = static_cast<int64_t>(steps) * D4S4_BYTES;
  auto row_of = [=](int row) { return static_cast<int64_t>(min(m0 + row, a.M - 1)); };
  auto col_of = [=](int col) { return static_cast<int64_t>(min(n0 + col, a.N - 1)); };
  auto emit = [=](int row, int col, float v) {
    const int m = m0 + row, n = n0 + col;
    if (m < a.M && n < a.N) store_scalar(a.out, static_cast<int64_t>(m) * a.N + n, v, a.out_kind);
  };
  if constexpr (DUMP) {
    q8_tile_run<true, COLS>(a.xq, x_row_bytes, a.w, w_row_bytes, steps, s, row_of, col_of, emit,
                            [=](int row, int col, int block, int dot) {
                              const int m = m0 + row, n = n0 + col;
                              if (m < a.M && n < a.N) dots[(static_cast<int64_t>(m) * a.N + n) * (a.K / 32) + block] = dot;
                            });
  } else {
    q8_tile_run<false, COLS>(a.xq, x_row_bytes, a.w, w_row_bytes, steps, s, row_of, col_of, emit);
  }
}

int launch_q8_0(const void* xq, const uint8_t* w, void* out, int out_kind, int64_t M, int64_t K, int64_t N,
                hipStream_t stream) {
  if (!xq || !w || !out || M <= 0 || M > (1 << 20) || K <= 0 || (K % 128) != 0 || N <= 0 || N > (1 << 24) ||
      out_kind < KIND_F32 || out_kind > KIND_F16) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  MmqArgs a{static_cast<const uint8_t*>(xq), w, out, out_kind, static_cast<int>(M), static_cast<int>(K),
            static_cast<int>(N)};
  // the tile width by the rule of the Q6_K launch: 64-wide tiles where they fill the rounds of resident
  // workgroups better
  const int64_t m_tiles = (M + BM - 1) / BM;
  const int64_t wide = m_tiles * ((N + 127) / 128), narrow = m_tiles * ((N + 63) / 64);
  const int64_t slots = 2 * 256;
  auto fill = [&](int64_t tiles) { return static_cast<double>(tiles) / static_cast<double>((tiles + slots - 1) / slots * slots); };
  if (Q6_TILE_CHOICE(fill(wide), fill(narrow))) {
    const dim3 grid(static_cast<unsigned>(m_tiles), static_cast<unsigned>((N + 63) / 64));
    hipLaunchKernelGGL((mmq_q8_0_d4s4_kernel<false, 64>), grid, dim3(THREADS), sizeof(Q8Smem<64>), stream, a,
                       static_cast<int32_t*>(nullptr));
  } else {
    const dim3 grid(static_cast<unsigned>(m_tiles), static_cast<unsigned>((N + BN - 1) / BN));
    hipLaunchKernelGGL((mmq_q8_0_d4s4_kernel<false, 128>), grid, dim3(THREADS), sizeof(Q8Smem<128>), stream, a,
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
  return launch_q4_tile<DenseQ5, false, 2>(a, stream);
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

// hipEngine's scheduling variants of the same GEMMs (gguf_k_mmq_prefill.hip:2565-2578 "pipe" and "mb4",
// :2315-2366 "direct_dp4a"): one kernel form here, the same results.
DEFINE_MMQ_Q5(hipengine_gguf_q5_k_mmq32_pipe_q8_1_d4s4_f32_bf16_bf16_out, KIND_BF16)
DEFINE_MMQ_Q5(hipengine_gguf_q5_k_mmq32_mb4_q8_1_d4s4_f32_bf16_bf16_out, KIND_BF16)
DEFINE_MMQ_Q5(hipengine_gguf_q5_k_mmq32_direct_dp4a_q8_1_d4s4_f32_bf16_bf16_out, KIND_BF16)
DEFINE_MMQ_Q5(hipengine_gguf_q5_k_mmq32_direct_dp4a_q8_1_d4s4_f32_bf16_f32_out, KIND_F32)
DEFINE_MMQ_Q6(hipengine_gguf_q6_k_mmq32_pipe_q8_1_d4s4_f32_bf16_bf16_out, KIND_BF16)
DEFINE_MMQ_Q6(hipengine_gguf_q6_k_mmq32_mb4_q8_1_d4s4_f32_bf16_bf16_out, KIND_BF16)

#define DEFINE_MMQ_Q8_0(SYMBOL, OKIND)                                                                      \
  extern "C" int SYMBOL(const void* xq, const uint8_t* qweight, void* out, int64_t rows, int64_t in_features, \
                        int64_t out_features, hipStream_t stream) {                                         \
    return launch_q8_0(xq, qweight, out, OKIND, rows, in_features, out_features, stream);                   \
  }

DEFINE_MMQ_Q8_0(hipengine_gguf_q8_0_mmq32_q8_1_d4s4_f32_bf16_f32_out, KIND_F32)
DEFINE_MMQ_Q8_0(hipengine_gguf_q8_0_mmq32_q8_1_d4s4_f32_bf16_bf16_out, KIND_BF16)

// ---- verification: the int32 dots the MMQ kernels feed their float32 combine with ----

extern "C" int hipengine_gfx950_gguf_mmq_dots_i32(int32_t ggml_type, const void* xq, const uint8_t* qweight,
                                                  int32_t* dots, float* out, int64_t rows, int64_t in_features,
                                                  int64_t out_features, hipStream_t stream) {
  if (!xq || !qweight || !dots || !out || rows <= 0 || rows > (1 << 20) || in_features <= 0 ||
      (in_features % (ggml_type == GGML_Q8_0 ? 128 : QK_K)) != 0 || out_features <= 0 || out_features > (1 << 24)) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  MmqArgs a{static_cast<const uint8_t*>(xq), qweight, out, KIND_F32, static_cast<int>(rows),
            static_cast<int>(in_features), static_cast<int>(out_features)};
  const dim3 grid(static_cast<unsigned>((rows + BM - 1) / BM), static_cast<unsigned>((out_features + BN - 1) / BN));
  if (ggml_type == GGML_Q4_K) {
    if ((out_features % 32) != 0) return static_cast<int>(hipErrorInvalidValue);
    const int rc = ensure_init();   // the LDS limit of this kernel
    if (rc != static_cast<int>(hipSuccess)) return rc;
    hipLaunchKernelGGL(mmq_tile_dump_kernel<DenseQ4>, grid, dim3(THREADS), sizeof(DenseQ4::Smem), stream, a, dots);
  } else if (ggml_type == GGML_Q5_K) {
    if ((out_features % 32) != 0) return static_cast<int>(hipErrorInvalidValue);
    hipLaunchKernelGGL(mmq_tile_dump_kernel<DenseQ5>, grid, dim3(THREADS), sizeof(DenseQ5::Smem), stream, a, dots);
  } else if (ggml_type == GGML_Q6_K) {
    hipLaunchKernelGGL((mmq_q6_k_d4s4_kernel<true, 128>), grid, dim3(THREADS), sizeof(Q6Smem<128>), stream, a, dots);
  } else if (ggml_type == GGML_Q8_0) {
    hipLaunchKernelGGL((mmq_q8_0_d4s4_kernel<true, 128>), grid, dim3(THREADS), sizeof(Q8Smem<128>), stream, a, dots);
  } else {
    return static_cast<int>(hipErrorInvalidValue);
  }
  return static_cast<int>(hipGetLastError());
}

// ---- prefill from bf16 activations: pack into the caller's workspace, then the MMQ ----

extern "C" int hipengine_gfx950_gguf_prefill_workspace_bytes(int32_t ggml_type, int64_t rows, int64_t in_features,
                                                             int64_t* bytes) {
  if (!bytes || rows <= 0 || in_features <= 0 || (in_features % (ggml_type == GGML_Q8_0 ? 128 : QK_K)) != 0 ||
      (ggml_type != GGML_Q4_K && ggml_type != GGML_Q5_K && ggml_type != GGML_Q6_K && ggml_type != GGML_Q8_0)) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  *bytes = rows * (in_features / 128) * (ggml_type == GGML_Q4_K ? DS4_BYTES : D4S4_BYTES);
  return static_cast<int>(hipSuccess);
}

// What the MMQ launch of a type refuses, checked before anything is enqueued (a call that is refused leaves
// nothing in the stream and writes nothing).
static bool prefill_shape_ok(int32_t ggml_type, const void* x, const uint8_t* qweight, const void* out, int32_t out_kind,
                             int64_t rows, int64_t in_features, int64_t out_features) {
  const bool type_ok = ggml_type == GGML_Q4_K || ggml_type == GGML_Q5_K || ggml_type == GGML_Q6_K || ggml_type == GGML_Q8_0;
  return type_ok && x && qweight && out && out_kind >= KIND_F32 && out_kind <= KIND_F16 && rows > 0 && in_features > 0 &&
         (in_features % (ggml_type == GGML_Q8_0 ? 128 : QK_K)) == 0 && out_features > 0 && out_features <= (1 << 24) &&
         ((ggml_type != GGML_Q4_K && ggml_type != GGML_Q5_K) || (out_features % 32) == 0);
}

// rows <= 2^20 of bf16 activations: pack into `workspace`, then the MMQ of the type
static int prefill_packed(int32_t ggml_type, const void* x, const uint8_t* qweight, void* out, int32_t out_kind, int64_t rows,
                          int64_t in_features, int64_t out_features, void* workspace, hipStream_t stream) {
  if (ggml_type == GGML_Q4_K) {
    const int prc = hipengine_gguf_q8_1_mmq_ds4_pack_bf16(x, workspace, rows, in_features, stream);
    if (prc != static_cast<int>(hipSuccess)) return prc;
    return launch_q4(workspace, qweight, out, out_kind, rows, in_features, out_features, 0, stream);
  }
  const int prc = hipengine_gguf_q8_1_d4s4_f32_quantize_bf16(x, workspace, rows, in_features, stream);
  if (prc != static_cast<int>(hipSuccess)) return prc;
  if (ggml_type == GGML_Q5_K) return launch_q5(workspace, qweight, out, out_kind, rows, in_features, out_features, stream);
  if (ggml_type == GGML_Q8_0) return launch_q8_0(workspace, qweight, out, out_kind, rows, in_features, out_features, stream);
  return launch_q6(workspace, qweight, out, out_kind, rows, in_features, out_features, stream);
}

extern "C" int hipengine_gfx950_gguf_prefill_bf16(int32_t ggml_type, const void* x, const uint8_t* qweight, void* out,
                                                  int32_t out_kind, int64_t rows, int64_t in_features,
                                                  int64_t out_features, void* workspace, int64_t workspace_bytes,
                                                  hipStream_t stream) {
  int64_t need = 0;
  const int rc = hipengine_gfx950_gguf_prefill_workspace_bytes(ggml_type, rows, in_features, &need);
  if (rc != static_cast<int>(hipSuccess)) return rc;
  if (!workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 15u) != 0 || rows > (1 << 20) ||
      !prefill_shape_ok(ggml_type, x, qweight, out, out_kind, rows, in_features, out_features)) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  return prefill_packed(ggml_type, x, qweight, out, out_kind, rows, in_features, out_features, workspace, stream);
}

// ---- the same with a pack buffer the library holds ----
//
// hipEngine's dense prefill entries take any number of rows and no workspace (gguf_q4_k_gemv.hip:1468-1493).  For
// them the packed activations of a chunk of rows go to a file-scope device array: two regions of 12 MiB, taken in
// turn by successive calls; a call walks its rows in chunks of up to 512 (pack, MMQ, pack, MMQ ... in stream
// order), so the weights are read once per 512 rows.  Nothing is allocated.  Calls that overlap on one device -
// more than two in flight on different streams - share a region and race.
namespace {
constexpr int64_t kPackRegionBytes = 12ll << 20;
constexpr int kPackRegions = 2;
constexpr int64_t kPackChunkRows = 512;
constexpr int64_t kPackMinChunkRows = 128;       // below this the chunks re-read the weights too often to pay
constexpr int kPackMaxDevices = 64;
__device__ __align__(256) uint8_t prefill_pack[kPackRegions * kPackRegionBytes];
std::atomic<uint8_t*> prefill_pack_ptr[kPackMaxDevices];
std::atomic<unsigned> prefill_next_region{0};
}  // namespace

int hipengine_gfx950::prefill_pack_setup(int device) {
  if (device < 0 || device >= kPackMaxDevices) return static_cast<int>(hipErrorInvalidDevice);
  if (prefill_pack_ptr[device].load(std::memory_order_acquire)) return static_cast<int>(hipSuccess);
  void* ptr = nullptr;
  const hipError_t err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(prefill_pack));
  if (err != hipSuccess) return static_cast<int>(err);
  if (!ptr) return static_cast<int>(hipErrorInvalidSymbol);
  prefill_pack_ptr[device].store(static_cast<uint8_t*>(ptr), std::memory_order_release);
  return static_cast<int>(hipSuccess);
}

bool hipengine_gfx950::prefill_library_buffer_takes(int ggml_type, int64_t rows, int64_t in_features, int64_t out_features) {
  if (rows < 32 || in_features <= 0 || (in_features % (ggml_type == GGML_Q8_0 ? 128 : QK_K)) != 0 || out_features <= 0 ||
      out_features > (1 << 24) || ((ggml_type == GGML_Q4_K || ggml_type == GGML_Q5_K) && (out_features % 32) != 0)) {
    return false;
  }
  const int64_t row_bytes = (in_features / 128) * (ggml_type == GGML_Q4_K ? DS4_BYTES : D4S4_BYTES);
  const int64_t fit = kPackRegionBytes / row_bytes;
  return fit >= kPackMinChunkRows || fit >= rows;
}

int hipengine_gfx950::prefill_bf16_library_buffer(int ggml_type, const void* x, const uint8_t* qweight, void* out, int out_kind,
                                                  int64_t rows, int64_t in_features, int64_t out_features,
                                                  hipStream_t stream) {
  if (!prefill_library_buffer_takes(ggml_type, rows, in_features, out_features) ||
      !prefill_shape_ok(ggml_type, x, qweight, out, out_kind, rows, in_features, out_features)) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  int device = -1;
  const hipError_t err = hipGetDevice(&device);
  if (err != hipSuccess) return static_cast<int>(err);
  if (device < 0 || device >= kPackMaxDevices) return static_cast<int>(hipErrorInvalidDevice);
  if (!prefill_pack_ptr[device].load(std::memory_order_acquire)) {   // first call on this device without hipengine_gfx950_init()
    const int rc = prefill_pack_setup(device);
    if (rc != static_cast<int>(hipSuccess)) return rc;
  }
  uint8_t* region = prefill_pack_ptr[device].load(std::memory_order_acquire) +
                    static_cast<int64_t>(prefill_next_region.fetch_add(1, std::memory_order_relaxed) % kPackRegions) * kPackRegionBytes;
  const int64_t row_bytes = (in_features / 128) * (ggml_type == GGML_Q4_K ? DS4_BYTES : D4S4_BYTES);
  int64_t chunk = kPackRegionBytes / row_bytes;
  chunk = chunk < kPackChunkRows ? chunk : kPackChunkRows;
  const int64_t out_elem = out_kind == KIND_F32 ? 4 : 2;
  for (int64_t r0 = 0; r0 < rows; r0 += chunk) {
    const int64_t n = rows - r0 < chunk ? rows - r0 : chunk;
    const int rc = prefill_packed(ggml_type, static_cast<const uint16_t*>(x) + r0 * in_features, qweight,
                                  static_cast<uint8_t*>(out) + r0 * out_features * out_elem, out_kind, n, in_features,
                                  out_features, region, stream);
    if (rc != static_cast<int>(hipSuccess)) return rc;
  }
  return static_cast<int>(hipSuccess);
}

int hipengine_gfx950::mmq_load() {
  // the Q4_K tile engine holds two copies of a K step's images: more than the 64 KiB a kernel may use unasked
  for (const void* fn : {reinterpret_cast<const void*>(mmq_q4_k_ds4_kernel<DenseQ4, false, 2>),
                         reinterpret_cast<const void*>(mmq_q4_k_ds4_kernel<DenseQ4, true, 2>),
                         reinterpret_cast<const void*>(mmq_tile_dump_kernel<DenseQ4>)}) {
    const hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize,
                                             static_cast<int>(sizeof(DenseQ4::Smem)));
    if (e != hipSuccess) return static_cast<int>(e);
  }
  hipFuncAttributes attr;
  return static_cast<int>(hipFuncGetAttributes(&attr, reinterpret_cast<const void*>(mmq_q6_k_d4s4_kernel<false, 128>)));
}
