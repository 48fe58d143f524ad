// C entry points of the dense q8_1 decode GEMV (Q4_K / Q6_K / Q8_0, batch 1..8)
// and the launch planner that maps a shape to a workgroup layout.
// The kernel body lives in gguf_gemv.hpp.

#include "gguf_gemv.hpp"
#include "gguf_gemv_run.hpp"
#include "gguf_gemv_stream.hpp"
#include "gguf_gemv_slab.hpp"
#include "gguf_gemv_pslab.hpp"
#include "gguf_init.hpp"

#include "../../include/hipengine_gfx950.h"
#include "../../include/hipengine_gfx950_tuning.h"

namespace {

using namespace hipengine_gfx950;

// Workgroup size cap per instantiation: the weight registers of a chunk
// (R*CB blocks) plus the per-batch-row activation reads have to fit the VGPR
// budget that the cap implies (128 registers at 1024 threads, 256 at 512).
template <int QT, int B, int R, int CB>
constexpr int gemv_max_threads() {
  return (R * CB * GemvTraits<QT>::REGS <= 64 && B <= 2) ? 1024 : 512;
}

template <int QT, int B, int R, int CB>
__global__ void __launch_bounds__((gemv_max_threads<QT, B, R, CB>())) gemv_kernel(GemvArgs a) {
  extern __shared__ __align__(16) uint8_t smem[];
  gemv_workgroup<QT, B, R, CB>(a, a.w, blockIdx.x * a.nrg * 16 * R, smem);
}

using KernelFn = void (*)(GemvArgs);

struct Variant {
  int b, r, cb;
  int max_threads;
  KernelFn fn;
};

#define GEMV_VARIANT(QT, B, R, CB) \
  Variant { B, R, CB, gemv_max_threads<QT, B, R, CB>(), gemv_kernel<QT, B, R, CB> }

#define GEMV_VARIANTS_FOR(QT)                                                              \
  GEMV_VARIANT(QT, 1, 1, 1), GEMV_VARIANT(QT, 1, 1, 2), GEMV_VARIANT(QT, 1, 1, 5),          \
  GEMV_VARIANT(QT, 1, 2, 1), GEMV_VARIANT(QT, 1, 2, 2), GEMV_VARIANT(QT, 1, 2, 5),          \
  GEMV_VARIANT(QT, 2, 1, 1), GEMV_VARIANT(QT, 2, 1, 2), GEMV_VARIANT(QT, 2, 1, 5),          \
  GEMV_VARIANT(QT, 2, 2, 1), GEMV_VARIANT(QT, 2, 2, 2), GEMV_VARIANT(QT, 2, 2, 5),          \
  GEMV_VARIANT(QT, 4, 1, 1), GEMV_VARIANT(QT, 4, 1, 2), GEMV_VARIANT(QT, 4, 1, 5),          \
  GEMV_VARIANT(QT, 4, 2, 1), GEMV_VARIANT(QT, 4, 2, 2), GEMV_VARIANT(QT, 4, 2, 5),          \
  GEMV_VARIANT(QT, 8, 1, 1), GEMV_VARIANT(QT, 8, 1, 2), GEMV_VARIANT(QT, 8, 1, 5),          \
  GEMV_VARIANT(QT, 8, 2, 1), GEMV_VARIANT(QT, 8, 2, 2), GEMV_VARIANT(QT, 8, 2, 5)

const Variant kQ4K[] = {GEMV_VARIANTS_FOR(GGML_Q4_K)};
const Variant kQ5K[] = {GEMV_VARIANTS_FOR(GGML_Q5_K)};
const Variant kQ6K[] = {GEMV_VARIANTS_FOR(GGML_Q6_K)};
const Variant kQ80[] = {GEMV_VARIANTS_FOR(GGML_Q8_0)};
constexpr int kVariants = 24;

const Variant* find_variant(int qt, int b, int r, int cb) {
  const Variant* table = qt == GGML_Q4_K ? kQ4K : qt == GGML_Q5_K ? kQ5K : qt == GGML_Q6_K ? kQ6K : qt == GGML_Q8_0 ? kQ80 : nullptr;
  if (!table) return nullptr;
  for (int i = 0; i < kVariants; ++i)
    if (table[i].b == b && table[i].r == r && table[i].cb == cb) return &table[i];
  return nullptr;
}


// ---- run form (whole rows per wave, contiguous block runs) -------------------

// XK >= 0 fixes the activation kind at compile time and promises that the two activation groups per
// thread fetched up front cover K (less prologue code to fetch cold), XK < 0 reads the kind from the
// arguments and takes any K.
template <int QT, int B, int G, int CB, int XK = -1>
__global__ void __launch_bounds__(512) gemv_run_kernel(GemvRunArgs a) {
  extern __shared__ __align__(16) uint8_t smem[];
  if constexpr (XK >= 0) a.x_kind = XK;
  gemv_run_workgroup<QT, B, G, CB, (XK >= 0)>(a, smem);
}

using RunKernelFn = void (*)(GemvRunArgs);

struct RunVariant {
  int b, g, cb;
  RunKernelFn fn;
  RunKernelFn by_kind[2];   // float32 and bf16 activations (null: use fn)
};

#define RUN_VARIANT(QT, B, G, CB) \
  RunVariant { B, G, CB, gemv_run_kernel<QT, B, G, CB>, {nullptr, nullptr} }
// the variants the default plan picks for K = 4096 and 5120 (4 rows per run, 5 loads per chunk)
#define RUN_VARIANT_BY_KIND(QT, B, G, CB)              \
  RunVariant { B, G, CB, gemv_run_kernel<QT, B, G, CB>, \
               {gemv_run_kernel<QT, B, G, CB, KIND_F32>, gemv_run_kernel<QT, B, G, CB, KIND_BF16>} }
#define RUN_VARIANTS_FOR(QT)                                                                        \
  RUN_VARIANT(QT, 1, 1, 1), RUN_VARIANT(QT, 1, 2, 1), RUN_VARIANT(QT, 1, 4, 1), RUN_VARIANT(QT, 1, 8, 1), \
  RUN_VARIANT(QT, 1, 1, 5), RUN_VARIANT(QT, 1, 2, 5), RUN_VARIANT_BY_KIND(QT, 1, 4, 5), RUN_VARIANT(QT, 1, 8, 5), \
  RUN_VARIANT(QT, 2, 1, 1), RUN_VARIANT(QT, 2, 2, 1), RUN_VARIANT(QT, 2, 4, 1), RUN_VARIANT(QT, 2, 8, 1), \
  RUN_VARIANT(QT, 2, 1, 5), RUN_VARIANT(QT, 2, 2, 5), RUN_VARIANT_BY_KIND(QT, 2, 4, 5), RUN_VARIANT(QT, 2, 8, 5)

const RunVariant kRunQ4K[] = {RUN_VARIANTS_FOR(GGML_Q4_K)};
const RunVariant kRunQ6K[] = {RUN_VARIANTS_FOR(GGML_Q6_K)};
const RunVariant kRunQ80[] = {RUN_VARIANTS_FOR(GGML_Q8_0)};
constexpr int kRunVariants = 16;

const RunVariant* find_run_variant(int qt, int b, int g, int cb) {
  const RunVariant* table = qt == GGML_Q4_K ? kRunQ4K : qt == GGML_Q6_K ? kRunQ6K : qt == GGML_Q8_0 ? kRunQ80 : nullptr;
  if (!table) return nullptr;
  for (int i = 0; i < kRunVariants; ++i)
    if (table[i].b == b && table[i].g == g && table[i].cb == cb) return &table[i];
  return nullptr;
}

constexpr size_t kMaxLds = 160 * 1024;   // LDS of one CU

// ---- slab form (Q4_K on the int8 MFMA, one workgroup per CU, waves split K) ----

// BPW = 1: up to 16 waves (K <= 4096); BPW = 2: up to 12 waves (K <= 6144), whose 64
// operand registers want the 170-register budget of a 768-thread bound.
template <int B, int BPW, int XK>
__global__ void __launch_bounds__(BPW == 1 ? 1024 : 768) gemv_slab_q4k_kernel(GemvSlabArgs a) {
  extern __shared__ __align__(16) uint8_t smem[];
  gemv_slab_q4k_workgroup<B, BPW, XK>(a, smem);
}

using SlabKernelFn = void (*)(GemvSlabArgs);
struct SlabVariant {
  int b, bpw;
  SlabKernelFn by_kind[4];
};
#define SLAB_VARIANT(B, BPW)                                                                            \
  SlabVariant { B, BPW, {gemv_slab_q4k_kernel<B, BPW, KIND_F32>, gemv_slab_q4k_kernel<B, BPW, KIND_BF16>, \
                         gemv_slab_q4k_kernel<B, BPW, KIND_F16>, gemv_slab_q4k_kernel<B, BPW, KIND_Q8_1>} }
const SlabVariant kSlab[] = {SLAB_VARIANT(1, 1), SLAB_VARIANT(1, 2), SLAB_VARIANT(2, 1), SLAB_VARIANT(2, 2),
                       SLAB_VARIANT(4, 1), SLAB_VARIANT(4, 2), SLAB_VARIANT(8, 1), SLAB_VARIANT(8, 2)};

struct SlabPlan {
  int b, bpw, waves, two_block_waves, rows_wg;
  bool ok;
};

// K <= 4096: one block per wave (up to 16 waves).  4352 <= K <= 6144: 12 waves, the first nb - 12 of them
// with two blocks, so that every SIMD gets three waves and (at K = 5120) five blocks.
SlabPlan default_slab_plan(int qt, int rows, int64_t K, int64_t N) {
  SlabPlan p{};
  const int nb = static_cast<int>(K / QK_K);
  p.b = rows <= 1 ? 1 : rows <= 2 ? 2 : rows <= 4 ? 4 : 8;
  p.bpw = nb <= 16 ? 1 : 2;
  p.waves = p.bpw == 1 ? nb : 12;
  p.two_block_waves = p.bpw == 1 ? 0 : nb - 12;
  const int64_t per_cu = (N + 255) / 256;
  p.rows_wg = static_cast<int>(per_cu < 1 ? 1 : per_cu > SLAB_MAX_ROWS ? SLAB_MAX_ROWS : per_cu);
  p.ok = qt == GGML_Q4_K && rows >= 1 && rows <= 8 && nb >= 4 && nb <= 24 &&
         gemv_slab_lds_bytes(p.b, p.waves, p.two_block_waves) <= 160 * 1024;
  return p;
}

int launch_gemv_slab(const void* x, int x_kind, const uint8_t* w, void* out, int out_kind, int rows, int64_t K,
                     int64_t N, const SlabPlan& p, hipStream_t stream, const void* residual = nullptr,
                     const void* gate = nullptr) {
  const int nb = static_cast<int>(K / QK_K);
  const SlabVariant* v = nullptr;
  for (const SlabVariant& c : kSlab)
    if (c.b == p.b && c.bpw == p.bpw) v = &c;
  if (!v || rows > p.b || x_kind < KIND_F32 || x_kind > KIND_Q8_1 || p.rows_wg < 1 || p.rows_wg > SLAB_MAX_ROWS ||
      p.waves < 1 || p.waves > (p.bpw == 1 ? 16 : 12) || p.two_block_waves < 0 || p.two_block_waves > p.waves ||
      (p.bpw == 1 && p.two_block_waves != 0) || p.waves + p.two_block_waves != nb || K > (1 << 20) ||
      N > (1 << 30)) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  const size_t lds = gemv_slab_lds_bytes(p.b, p.waves, p.two_block_waves);
  if (lds > 160 * 1024) return static_cast<int>(hipErrorInvalidValue);
  if (lds > 64 * 1024) {   // above the default dynamic limit: raised for every kernel by the library set-up
    const int rc = ensure_init();
    if (rc != static_cast<int>(hipSuccess)) return rc;
  }
  GemvSlabArgs a{x, w, out, x_kind, out_kind, rows, static_cast<int>(K), static_cast<int>(N), p.rows_wg, p.waves,
                 p.two_block_waves, residual, gate};
  const unsigned grid = static_cast<unsigned>((N + p.rows_wg - 1) / p.rows_wg);
  hipLaunchKernelGGL(v->by_kind[x_kind], dim3(grid), dim3(p.waves * 64), lds, stream, a);
  return static_cast<int>(hipGetLastError());
}

// ---- phased slab form (Q6_K / Q8_0, and Q4_K rows too long for the slab form, on the int8 MFMA; batch 3..8) ----

template <int QT, int B, bool PHASED, int XK>
__global__ void __launch_bounds__(768) gemv_pslab_kernel(GemvPslabArgs a) {
  extern __shared__ __align__(16) uint8_t smem[];
  gemv_pslab_workgroup<QT, B, PHASED, XK>(a, smem);
}

using PslabKernelFn = void (*)(GemvPslabArgs);
struct PslabVariant {
  int qt, b;
  bool phased;
  PslabKernelFn by_kind[4];
};
#define PSLAB_VARIANT(QT, B, P)                                                                              \
  PslabVariant { QT, B, P, {gemv_pslab_kernel<QT, B, P, KIND_F32>, gemv_pslab_kernel<QT, B, P, KIND_BF16>,   \
                            gemv_pslab_kernel<QT, B, P, KIND_F16>, gemv_pslab_kernel<QT, B, P, KIND_Q8_1>} }
const PslabVariant kPslab[] = {PSLAB_VARIANT(GGML_Q5_K, 4, false), PSLAB_VARIANT(GGML_Q5_K, 4, true),
                         PSLAB_VARIANT(GGML_Q5_K, 8, false), PSLAB_VARIANT(GGML_Q5_K, 8, true),
                         PSLAB_VARIANT(GGML_Q4_K, 4, false), PSLAB_VARIANT(GGML_Q4_K, 4, true),
                         PSLAB_VARIANT(GGML_Q4_K, 8, false), PSLAB_VARIANT(GGML_Q4_K, 8, true),
                         PSLAB_VARIANT(GGML_Q6_K, 4, false), PSLAB_VARIANT(GGML_Q6_K, 4, true),
                         PSLAB_VARIANT(GGML_Q6_K, 8, false), PSLAB_VARIANT(GGML_Q6_K, 8, true),
                         PSLAB_VARIANT(GGML_Q8_0, 4, false), PSLAB_VARIANT(GGML_Q8_0, 4, true),
                         PSLAB_VARIANT(GGML_Q8_0, 8, false), PSLAB_VARIANT(GGML_Q8_0, 8, true)};

struct PslabPlan {
  int b, waves, bpw_log2, phases, grid;
  bool ok;
};

size_t pslab_lds_bytes(int qt, int b, int waves, int bpw) {
  return static_cast<size_t>(waves) * (qt == GGML_Q6_K   ? pslab_wave_bytes<GGML_Q6_K>(b, bpw)
                                       : qt == GGML_Q4_K ? pslab_wave_bytes<GGML_Q4_K>(b, bpw)
                                       : qt == GGML_Q5_K ? pslab_wave_bytes<GGML_Q5_K>(b, bpw)
                                                         : pslab_wave_bytes<GGML_Q8_0>(b, bpw));
}

int64_t pslab_row_bytes(int qt, int nb) {
  return static_cast<int64_t>(nb) * (qt == GGML_Q6_K   ? Q6_K_BYTES
                                     : qt == GGML_Q4_K ? Q4_K_BYTES
                                     : qt == GGML_Q5_K ? Q5_K_BYTES
                                                       : 8 * Q8_0_BYTES);
}

int pslab_grid(int64_t N, int phases) {
  // one phase: a workgroup per CU walks its share of the rows group by group; several phases: a
  // workgroup has one group of at most 96 rows
  const int64_t groups = (N + PSLAB_GROUP_ROWS - 1) / PSLAB_GROUP_ROWS;
  const int64_t per_cu = N < 256 ? N : 256;
  return static_cast<int>(phases == 1 ? per_cu : (groups > per_cu ? groups : per_cu));
}

// Waves and blocks per wave: the split of K/256 blocks over W <= 12 waves x bpw in {1, 2, 4} slots x phases
// that loads the four SIMDs most evenly, preferring a single phase (activations quantized once) and more
// waves.
PslabPlan default_pslab_plan(int qt, int rows, int64_t K, int64_t N, const void* w) {
  PslabPlan p{};
  const int nb = static_cast<int>(K / QK_K);
  const int64_t row_bytes = pslab_row_bytes(qt, nb);
  if ((qt != GGML_Q4_K && qt != GGML_Q5_K && qt != GGML_Q6_K && qt != GGML_Q8_0) || rows < 1 || rows > 8 || nb < 8 || (nb & 1) != 0 ||
      (reinterpret_cast<uintptr_t>(w) & 3u) != 0 || N < 1 || row_bytes >= (1 << 24) || N * row_bytes > 0xFFFF0000ll) {
    return p;
  }
  p.b = rows <= 4 ? 4 : 8;
  float best = -1.0f;
  for (int waves = 12; waves >= 6; --waves) {
    for (int bl2 = 0; bl2 <= 2; ++bl2) {
      const int bpw = 1 << bl2;
      if (waves > nb || pslab_lds_bytes(qt, p.b, waves, bpw) > kMaxLds) continue;
      const int phases = (nb + waves * bpw - 1) / (waves * bpw);
      // wave w owns blocks w, w + waves, ...: the SIMD (w % 4) with the most blocks sets the pace
      int simd_blocks[4] = {0, 0, 0, 0};
      for (int w = 0; w < waves; ++w) simd_blocks[w & 3] += (nb - w + waves - 1) / waves;
      int worst = 0;
      for (int v : simd_blocks) worst = v > worst ? v : worst;
      const float score = static_cast<float>(nb) / static_cast<float>(4 * worst) -
                          0.02f * static_cast<float>(12 - waves) + (phases == 1 ? 0.05f : 0.0f) - 0.001f * bl2;
      if (score > best) {
        best = score;
        p.waves = waves; p.bpw_log2 = bl2; p.phases = phases;
      }
    }
  }
  if (best < 0.0f) return p;
  p.grid = pslab_grid(N, p.phases);
  p.ok = true;
  return p;
}

int launch_gemv_pslab(int qt, const void* x, int x_kind, const uint8_t* w, void* out, int out_kind, int rows,
                      int64_t K, int64_t N, const PslabPlan& p, hipStream_t stream, const void* residual = nullptr,
                      const void* gate = nullptr) {
  const int nb = static_cast<int>(K / QK_K);
  const int bpw = 1 << p.bpw_log2;
  const int64_t row_bytes = pslab_row_bytes(qt, nb);
  const PslabVariant* v = nullptr;
  for (const PslabVariant& c : kPslab)
    if (c.qt == qt && c.b == p.b && c.phased == (p.phases > 1)) v = &c;
  if (!v || rows < 1 || rows > p.b || x_kind < KIND_F32 || x_kind > KIND_Q8_1 || p.waves < 1 || p.waves > 12 ||
      p.bpw_log2 < 0 || p.bpw_log2 > 2 || p.waves > nb || (nb & 1) != 0 ||
      p.phases != (nb + p.waves * bpw - 1) / (p.waves * bpw) || p.grid < 1 ||
      (p.phases > 1 && static_cast<int64_t>(p.grid) * PSLAB_GROUP_ROWS < N) ||
      (reinterpret_cast<uintptr_t>(w) & 3u) != 0 || row_bytes >= (1 << 24) || N * row_bytes > 0xFFFF0000ll) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  const size_t lds = pslab_lds_bytes(qt, p.b, p.waves, bpw);
  if (lds > kMaxLds) return static_cast<int>(hipErrorInvalidValue);
  if (lds > 64 * 1024) {
    const int rc = ensure_init();
    if (rc != static_cast<int>(hipSuccess)) return rc;
  }
  GemvPslabArgs a{};
  a.x = x; a.w = w; a.out = out; a.residual = residual; a.gate = gate;
  a.x_kind = x_kind; a.out_kind = out_kind; a.rows = rows;
  a.K = static_cast<int>(K); a.N = static_cast<int>(N);
  a.waves = p.waves; a.bpw_log2 = p.bpw_log2; a.phases = p.phases;
  a.base_rows = static_cast<int>(N / p.grid);
  a.w_bytes = static_cast<uint32_t>((N * row_bytes + 3) & ~3ll);
  hipLaunchKernelGGL(v->by_kind[x_kind], dim3(static_cast<unsigned>(p.grid)), dim3(p.waves * 64), lds, stream, a);
  return static_cast<int>(hipGetLastError());
}

int gcd_int(int a, int b) { return b == 0 ? a : gcd_int(b, a % b); }

struct RunPlan {
  int b, g, cb, waves;
  bool ok;
};

// The run form applies when a whole number of rows fills a whole number of
// 16-block wave loads with at most 8 rows, the batch is 1 or 2 and the
// quantized activations of the whole K fit in LDS.
RunPlan default_run_plan(int qt, int rows, int64_t K, int64_t N) {
  RunPlan p{};
  const int nb = static_cast<int>(K / QK_K);
  p.b = rows <= 1 ? 1 : 2;
  p.g = 16 / gcd_int(nb, 16);
  const int m = p.g * nb / 16;
  p.cb = m >= 2 ? 5 : 1;
  // Every workgroup quantizes the whole activation row (nb*32 lane tasks of 8 values), so
  // the workgroup is sized for at most ~2 of them per thread rather than for a large
  // grid: 13.5 -> 6.7 us at K=5120, N=1024 with 8 waves instead of 1.
  const int want = (nb * 32 + 127) / 128;
  p.waves = want >= 5 ? 8 : want >= 3 ? 4 : 2;
  p.ok = rows <= 2 && p.g <= 8 && gemv_run_lds_bytes(qt, p.b, static_cast<int>(K)) <= 64 * 1024 &&
         find_run_variant(qt, p.b, p.g, p.cb) != nullptr;
  return p;
}

int launch_gemv_run(int qt, const void* x, int x_kind, const uint8_t* w, void* out, int out_kind, int rows, int64_t K,
                    int64_t N, const RunPlan& p, hipStream_t stream) {
  const RunVariant* v = find_run_variant(qt, p.b, p.g, p.cb);
  const int nb = static_cast<int>(K / QK_K);
  if (!v || p.waves < 1 || p.waves > 8 || (p.g * nb) % 16 != 0 || rows > p.b) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  const size_t lds = gemv_run_lds_bytes(qt, p.b, static_cast<int>(K));
  if (lds > 64 * 1024) return static_cast<int>(hipErrorInvalidValue);
  GemvRunArgs a;
  a.x = x; a.w = w; a.out = out;
  a.x_kind = x_kind; a.out_kind = out_kind;
  a.rows = rows; a.K = static_cast<int>(K); a.N = static_cast<int>(N);
  a.waves = p.waves;
  const int64_t runs = (N + p.g - 1) / p.g;
  const unsigned grid = static_cast<unsigned>((runs + p.waves - 1) / p.waves);
  const bool up_front = nb * 8 <= 2 * p.waves * 16;
  const RunKernelFn fn =
      up_front && (x_kind == KIND_F32 || x_kind == KIND_BF16) && v->by_kind[x_kind] ? v->by_kind[x_kind] : v->fn;
  hipLaunchKernelGGL(fn, dim3(grid), dim3(p.waves * 64), lds, stream, a);
  return static_cast<int>(hipGetLastError());
}


// ---- stream form (resident waves, ring of loads in flight) --------------------

// Batch 1 kernels fit 170 registers and may run 12 waves per workgroup, which lets the
// planner pick a wave count that divides the rows evenly.
template <int B>
constexpr int stream_max_threads() {
  return B == 1 ? 768 : 512;
}

template <int QT, int B, int D, int S, int XK = -1, int FUSE = FUSE_NONE>
__global__ void __launch_bounds__((stream_max_threads<B>())) gemv_stream_kernel(GemvStreamArgs a) {
  extern __shared__ __align__(16) uint8_t smem[];
  gemv_stream_workgroup<QT, B, D, S, XK, FUSE>(a, smem);
}

using StreamKernelFn = void (*)(GemvStreamArgs);

// `long_k`: the instantiation that fetches five activation groups (of 8 values) per thread
// up front (batch 1 only); the other fetches two (batch 1, 2) or one (batch 4, 8).
// `fuse`: plain projection, gate/up pair with SiLU, or projection plus residual.
struct StreamVariant {
  int qt, b, d;
  int s;         // activation groups (of 8 values) per thread fetched up front
  bool long_k;
  int fuse;
  StreamKernelFn fn;
  StreamKernelFn by_kind[4];   // instantiations with the activation kind fixed (null: use fn)
};

#define STREAM_VARIANT(QT, B, D) \
  StreamVariant { QT, B, D, (B <= 2 ? 2 : 1), false, FUSE_NONE, gemv_stream_kernel<QT, B, D, (B <= 2 ? 2 : 1)>, {nullptr, nullptr, nullptr, nullptr} }
#define STREAM_VARIANT_BY_KIND(QT, B, D, S, LONG_K)                                                      \
  StreamVariant { QT, B, D, S, LONG_K, FUSE_NONE, gemv_stream_kernel<QT, B, D, S>,                        \
                  {gemv_stream_kernel<QT, B, D, S, KIND_F32>, gemv_stream_kernel<QT, B, D, S, KIND_BF16>, \
                   gemv_stream_kernel<QT, B, D, S, KIND_F16>, gemv_stream_kernel<QT, B, D, S, KIND_Q8_1>} }
// fused epilogues: float32 and bf16 activations get instantiations of their own, the other kinds the generic one
#define STREAM_VARIANT_FUSED_D(QT, B, D, S, LONG_K, FUSE)                                                        \
  StreamVariant { QT, B, D, S, LONG_K, FUSE, gemv_stream_kernel<QT, B, D, S, -1, FUSE>,                           \
                  {gemv_stream_kernel<QT, B, D, S, KIND_F32, FUSE>, gemv_stream_kernel<QT, B, D, S, KIND_BF16, FUSE>, \
                   nullptr, nullptr} }
#define STREAM_VARIANT_FUSED(QT, B, S, LONG_K, FUSE) STREAM_VARIANT_FUSED_D(QT, B, 3, S, LONG_K, FUSE)

const StreamVariant kStream[] = {
    STREAM_VARIANT_BY_KIND(GGML_Q4_K, 1, 3, 2, false), STREAM_VARIANT_BY_KIND(GGML_Q4_K, 2, 3, 2, false),
    STREAM_VARIANT_BY_KIND(GGML_Q4_K, 1, 2, 2, false),
    STREAM_VARIANT_BY_KIND(GGML_Q6_K, 1, 3, 2, false), STREAM_VARIANT_BY_KIND(GGML_Q6_K, 2, 3, 2, false),
    STREAM_VARIANT_BY_KIND(GGML_Q8_0, 1, 3, 2, false), STREAM_VARIANT_BY_KIND(GGML_Q8_0, 2, 3, 2, false),
    STREAM_VARIANT_BY_KIND(GGML_Q5_K, 1, 3, 2, false), STREAM_VARIANT_BY_KIND(GGML_Q5_K, 2, 3, 2, false),
    STREAM_VARIANT_BY_KIND(GGML_Q5_K, 1, 3, 5, true),
    STREAM_VARIANT_BY_KIND(GGML_Q4_K, 1, 3, 5, true), STREAM_VARIANT_BY_KIND(GGML_Q6_K, 1, 3, 5, true),
    STREAM_VARIANT_BY_KIND(GGML_Q8_0, 1, 3, 5, true),
    STREAM_VARIANT_BY_KIND(GGML_Q4_K, 2, 3, 5, true), STREAM_VARIANT_BY_KIND(GGML_Q6_K, 2, 3, 5, true),
    STREAM_VARIANT(GGML_Q4_K, 4, 3), STREAM_VARIANT(GGML_Q4_K, 8, 3), STREAM_VARIANT(GGML_Q6_K, 4, 3),
    STREAM_VARIANT(GGML_Q6_K, 8, 3), STREAM_VARIANT(GGML_Q8_0, 4, 3), STREAM_VARIANT(GGML_Q8_0, 8, 3),
    // gate/up pair with SiLU (Q4_K) and projection + residual (Q4_K, Q6_K), batch 1 and 2
    STREAM_VARIANT_FUSED(GGML_Q4_K, 1, 2, false, FUSE_PAIR), STREAM_VARIANT_FUSED(GGML_Q4_K, 2, 2, false, FUSE_PAIR),
    STREAM_VARIANT_FUSED(GGML_Q4_K, 1, 2, false, FUSE_RESIDUAL), STREAM_VARIANT_FUSED(GGML_Q4_K, 2, 2, false, FUSE_RESIDUAL),
    STREAM_VARIANT_FUSED(GGML_Q6_K, 1, 2, false, FUSE_RESIDUAL), STREAM_VARIANT_FUSED(GGML_Q6_K, 2, 2, false, FUSE_RESIDUAL),
    STREAM_VARIANT_FUSED(GGML_Q4_K, 1, 5, true, FUSE_RESIDUAL), STREAM_VARIANT_FUSED(GGML_Q6_K, 1, 5, true, FUSE_RESIDUAL),
    // the tall Q4_K shape at batch 1 on a ring of two (see tuned_stream_plan)
    STREAM_VARIANT_FUSED_D(GGML_Q4_K, 1, 2, 2, false, FUSE_PAIR), STREAM_VARIANT_FUSED_D(GGML_Q4_K, 1, 2, 2, false, FUSE_RESIDUAL),
};

// The variant a launch takes: of those for (type, batch bucket, ring depth, epilogue), the one with the fewest
// up-front groups per thread that still cover K with this many waves (nb*8 groups, 16 teams per wave);
// if none does, the one with the most (its generic kernel loops over the rest).
const StreamVariant* pick_stream_variant(int qt, int b, int d, int fuse, int nb, int waves) {
  const StreamVariant* best = nullptr;
  bool best_covers = false;
  for (const StreamVariant& v : kStream) {
    if (v.qt != qt || v.b != b || v.d != d || v.fuse != fuse) continue;
    const bool covers = nb * 8 <= v.s * waves * 16;
    if (!best || (covers && (!best_covers || v.s < best->s)) || (!covers && !best_covers && v.s > best->s)) {
      best = &v;
      best_covers = covers;
    }
  }
  return best;
}

const StreamVariant* find_stream_variant(int qt, int b, int d, bool long_k = false, int fuse = FUSE_NONE) {
  const StreamVariant* fallback = nullptr;
  for (const StreamVariant& v : kStream) {
    if (v.qt != qt || v.b != b || v.d != d || v.fuse != fuse) continue;
    if (v.long_k == long_k) return &v;
    if (!v.long_k) fallback = &v;
  }
  return fallback;
}

int batch_bucket(int rows) { return rows <= 1 ? 1 : rows <= 2 ? 2 : rows <= 4 ? 4 : 8; }

struct StreamPlan {
  int b, d, waves, waves_total;
  bool ok;
};

constexpr int kComputeUnits = 256;   // MI355X

// The stream form applies to K >= 4096 (a 16-block load then spans at most two
// rows), batch <= 2, when every resident wave gets at least a few loads.
StreamPlan default_stream_plan(int qt, int rows, int64_t K, int64_t N) {
  StreamPlan p{};
  const int nb = static_cast<int>(K / QK_K);
  p.b = batch_bucket(rows);
  p.d = 3;
  p.waves = 8;
  const int64_t total_loads = N * nb / 16;
  // 8 resident waves per CU once every wave gets 3 loads or more, else 4 per CU
  p.waves_total = total_loads >= 6144 ? kComputeUnits * 8 : kComputeUnits * 4;
  if (p.b == 1 && total_loads >= 6144) {
    // whole rows per wave: 8, 10 or 12 waves per CU, whichever splits the rows most
    // evenly (N = 5120: 2.5 rows per wave at 8, exactly 2 at 10)
    double best = 1e9;
    for (int w = 8; w <= 12; w += 2) {
      const int64_t wt = static_cast<int64_t>(kComputeUnits) * w;
      if (wt > N) break;
      const double imbalance = static_cast<double>((N + wt - 1) / wt) * wt / static_cast<double>(N);
      if (imbalance < best - 0.1) { best = imbalance; p.waves = w; p.waves_total = static_cast<int>(wt); }
    }
  }
  // every wave should get the ring's three loads; Q4_K at batch 1 still beats the slab form with two
  // (5120 x 5120 on 10 waves per CU: 6.7 us against 7.8)
  const int min_loads = (qt == GGML_Q4_K && p.b == 1) ? 2 : 3;
  p.ok = rows <= 8 && nb >= 16 && total_loads >= min_loads * static_cast<int64_t>(p.waves_total) &&
         N >= p.waves_total && gemv_run_lds_bytes(qt, p.b, static_cast<int>(K)) <= kMaxLds &&
         find_stream_variant(qt, p.b, p.d) != nullptr;
  return p;
}

// The plan the entry points launch with.  A tall Q4_K matrix at batch 1 (every wave of a 12-per-CU grid still
// gets six loads: the 17408 x 5120 gate/up shape) runs 12 waves per CU with two loads in flight each:
// measured 12.1 us against 12.3 for 8 waves with three (the same bytes in flight, rows split 6/5
// instead of 9/8).
// The fused forms take the same plan as the plain projection, so that their float32 sums are the same.
StreamPlan tuned_stream_plan(int qt, int rows, int64_t K, int64_t N) {
  StreamPlan p = default_stream_plan(qt, rows, K, N);
  const int64_t nb = K / QK_K;
  const int64_t wt = static_cast<int64_t>(kComputeUnits) * 12;
  if (p.ok && qt == GGML_Q4_K && p.b == 1 && nb <= 32 && N * nb / 16 >= 6 * wt && find_stream_variant(qt, 1, 2) != nullptr &&
      find_stream_variant(qt, 1, 2, false, FUSE_PAIR) != nullptr && find_stream_variant(qt, 1, 2, false, FUSE_RESIDUAL) != nullptr) {
    p.d = 2;
    p.waves = 12;
    p.waves_total = static_cast<int>(wt);
  }
  return p;
}

struct StreamFusion {
  int fuse = FUSE_NONE;
  const uint8_t* w_up = nullptr;
  const void* residual = nullptr;
  int round_mid = 0;
};

int launch_gemv_stream(int qt, const void* x, int x_kind, const uint8_t* w, void* out, int out_kind, int rows,
                       int64_t K, int64_t N, const StreamPlan& p, hipStream_t stream,
                       const StreamFusion& fusion = StreamFusion()) {
  const int nb = static_cast<int>(K / QK_K);
  const StreamVariant* v = p.waves > 0 ? pick_stream_variant(qt, p.b, p.d, fusion.fuse, nb, p.waves) : nullptr;
  if (!v || nb < 16 || rows > p.b || p.waves < 1 || p.waves > (p.b == 1 ? 12 : 8) || p.waves_total < p.waves ||
      (p.waves_total % p.waves) != 0 || p.waves_total > N) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  size_t lds = gemv_run_lds_bytes(qt, p.b, static_cast<int>(K));
  if (fusion.fuse == FUSE_PAIR) {
    // gate results wait per wave; a wave may hold at most STREAM_PAIR_MAX_ROWS rows
    if (!fusion.w_up || (N + p.waves_total - 1) / p.waves_total > STREAM_PAIR_MAX_ROWS) return static_cast<int>(hipErrorInvalidValue);
    lds += static_cast<size_t>(p.waves) * p.b * STREAM_PAIR_MAX_ROWS * sizeof(float);
  }
  if (fusion.fuse == FUSE_RESIDUAL && !fusion.residual) return static_cast<int>(hipErrorInvalidValue);
  if (lds > kMaxLds) return static_cast<int>(hipErrorInvalidValue);
  // the kind-specialised kernels stage the whole row from the groups fetched up front
  const bool up_front = nb * 8 <= v->s * p.waves * 16;
  const StreamKernelFn fn =
      (up_front && x_kind >= KIND_F32 && x_kind <= KIND_Q8_1 && v->by_kind[x_kind]) ? v->by_kind[x_kind] : v->fn;
  if (lds > 64 * 1024) {
    const int rc = ensure_init();
    if (rc != static_cast<int>(hipSuccess)) return rc;
  }
  GemvStreamArgs a;
  a.x = x; a.w = w; a.out = out;
  a.x_kind = x_kind; a.out_kind = out_kind;
  a.rows = rows; a.K = static_cast<int>(K); a.N = static_cast<int>(N);
  a.waves = p.waves; a.waves_total = p.waves_total;
  a.base_rows = static_cast<int>(N / p.waves_total);
  a.w_up = fusion.w_up; a.residual = fusion.residual; a.round_mid = fusion.round_mid;
  hipLaunchKernelGGL(fn, dim3(p.waves_total / p.waves), dim3(p.waves * 64), lds, stream, a);
  return static_cast<int>(hipGetLastError());
}

struct Plan {
  int b, r, cb, ks, nrg;
};

// Default layout for a shape.  ks K-slices of CB blocks each cover one chunk;
// the row-group count is lowered until the launch has at least ~2 workgroups
// per CU (256 CUs) or reaches one row group.
Plan default_plan(int qt, int rows, int64_t K, int64_t N) {
  Plan p;
  const int nb = static_cast<int>(K / QK_K);
  p.b = batch_bucket(rows);
  p.r = p.b == 4 ? 2 : 1;
  p.ks = nb >= 4 ? 4 : nb;
  const int per_wave = (nb + p.ks - 1) / p.ks;
  p.cb = per_wave >= 5 ? 5 : per_wave >= 2 ? 2 : 1;
  if (p.r == 2 && p.cb > 2) p.cb = 2;   // keep R*CB blocks of weights within the register budget
  const Variant* v = find_variant(qt, p.b, p.r, p.cb);
  const int max_threads = v ? v->max_threads : 512;
  int nrg = max_threads / 64 / p.ks;
  if (nrg < 1) nrg = 1;
  while (nrg > 1 && (N + nrg * 16 * p.r - 1) / (nrg * 16 * p.r) < 512) nrg >>= 1;
  p.nrg = nrg;
  return p;
}

// The kernel form a batch of `chunk` <= 8 rows takes, and the rows of it that go in one launch.
enum GemvForm { FORM_ROW_STRIDED = 0, FORM_RUN = 1, FORM_STREAM = 2, FORM_SLAB = 3, FORM_PSLAB = 4 };

// Q4_K, K <= 6144: the int8 MFMA slab form wins for batches of 3 and more; at batch 2 when a slab is a single
// 32-row step (N <= 8192); at batch 1 only below 4096 rows (above, the stream form is ~1 us faster) or where
// the stream form does not apply.  Measured on MI355X.
bool slab_preferred(int qt, int chunk, int64_t K, int64_t N, const SlabPlan& sl) {
  if (!sl.ok) return false;
  if (chunk >= 3) return true;
  if (chunk == 2) return sl.rows_wg <= 32;
  return sl.rows_wg < 16 || (sl.rows_wg <= 32 && !default_stream_plan(qt, chunk, K, N).ok);
}

GemvForm pick_form(int qt, int& chunk, int64_t K, int64_t N, const void* w) {
  const SlabPlan sl = default_slab_plan(qt, chunk, K, N);
  const PslabPlan pp = default_pslab_plan(qt, chunk, K, N, w);
  // a batch of 5..8 whose quantized activations do not fit the LDS of any form that takes it whole
  // goes as two batches of at most 4, which do
  if (chunk > 4 && !sl.ok && !pp.ok && !default_stream_plan(qt, chunk, K, N).ok &&
      default_stream_plan(qt, 4, K, N).ok) {
    chunk = 4;
  }
  if (slab_preferred(qt, chunk, K, N, sl)) return FORM_SLAB;
  // the other types (and Q4_K with K > 6144), batch 3..8: the phased slab form on the int8 MFMA
  if (chunk >= 3 && default_pslab_plan(qt, chunk, K, N, w).ok) {
    return FORM_PSLAB;
  }
  if (default_stream_plan(qt, chunk, K, N).ok) return FORM_STREAM;
  if (default_run_plan(qt, chunk, K, N).ok) return FORM_RUN;
  return FORM_ROW_STRIDED;
}

int launch_gemv(int qt, const void* x, int x_kind, const uint8_t* w, void* out, int out_kind, int64_t rows, int64_t K,
                int64_t N, const Plan* forced, hipStream_t stream) {
  if (!x || !w || !out || rows <= 0 || K <= 0 || N <= 0 || (K % QK_K) != 0 || K > (1 << 24) || N > (1 << 30)) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  const int64_t x_row_bytes = x_kind == KIND_Q8_1 ? K / 32 * Q8_1_BYTES : K * (x_kind == KIND_F32 ? 4 : 2);
  const int64_t out_elem = out_kind == KIND_F32 ? 4 : 2;
  for (int64_t r0 = 0; r0 < rows;) {
    int chunk = static_cast<int>(rows - r0 < 8 ? rows - r0 : 8);
    const GemvForm form = forced ? FORM_ROW_STRIDED : pick_form(qt, chunk, K, N, w);
    const int64_t next_r0 = r0 + chunk;
    const void* xr = static_cast<const uint8_t*>(x) + r0 * x_row_bytes;
    void* outr = static_cast<uint8_t*>(out) + r0 * N * out_elem;
    if (form != FORM_ROW_STRIDED) {
      int rc;
      if (form == FORM_SLAB) {
        rc = launch_gemv_slab(xr, x_kind, w, outr, out_kind, chunk, K, N, default_slab_plan(qt, chunk, K, N), stream);
      } else if (form == FORM_PSLAB) {
        rc = launch_gemv_pslab(qt, xr, x_kind, w, outr, out_kind, chunk, K, N, default_pslab_plan(qt, chunk, K, N, w),
                               stream);
      } else if (form == FORM_STREAM) {
        rc = launch_gemv_stream(qt, xr, x_kind, w, outr, out_kind, chunk, K, N, tuned_stream_plan(qt, chunk, K, N),
                                stream);
      } else {
        rc = launch_gemv_run(qt, xr, x_kind, w, outr, out_kind, chunk, K, N, default_run_plan(qt, chunk, K, N), stream);
      }
      if (rc != static_cast<int>(hipSuccess)) return rc;
      r0 = next_r0;
      continue;
    }
    Plan p = forced ? *forced : default_plan(qt, chunk, K, N);
    if (forced) p.b = batch_bucket(chunk);
    const Variant* v = find_variant(qt, p.b, p.r, p.cb);
    if (!v || p.ks < 1 || p.nrg < 1 || p.ks * p.nrg * 64 > v->max_threads) {
      return static_cast<int>(hipErrorInvalidValue);
    }
    GemvArgs a;
    a.x = static_cast<const uint8_t*>(x) + r0 * x_row_bytes;
    a.w = w;
    a.out = static_cast<uint8_t*>(out) + r0 * N * out_elem;
    a.x_kind = x_kind;
    a.out_kind = out_kind;
    a.rows = chunk;
    a.K = static_cast<int>(K);
    a.N = static_cast<int>(N);
    a.ks = p.ks;
    a.nrg = p.nrg;
    const int rows_wg = p.nrg * 16 * p.r;
    const unsigned grid = static_cast<unsigned>((N + rows_wg - 1) / rows_wg);
    const size_t lds = gemv_lds_bytes(qt, p.b, p.r, p.cb, p.ks, p.nrg);
    if (lds > 64 * 1024) return static_cast<int>(hipErrorInvalidValue);
    hipLaunchKernelGGL(v->fn, dim3(grid), dim3(p.ks * p.nrg * 64), lds, stream, a);
    const hipError_t err = hipGetLastError();
    if (err != hipSuccess) return static_cast<int>(err);
    r0 = next_r0;
  }
  return static_cast<int>(hipSuccess);
}

}  // namespace

// Every slab, phased slab and stream kernel may be launched with more dynamic LDS than the 64 KB a kernel
// gets by default; the limit is raised for all of them here, once per device, so that no launch has to.
int hipengine_gfx950::gemv_raise_lds_limits() {
  auto raise = [](const void* fn) {
    return fn ? hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(kMaxLds))
              : hipSuccess;
  };
  for (const SlabVariant& v : kSlab)
    for (const SlabKernelFn fn : v.by_kind) {
      const hipError_t e = raise(reinterpret_cast<const void*>(fn));
      if (e != hipSuccess) return static_cast<int>(e);
    }
  for (const PslabVariant& v : kPslab)
    for (const PslabKernelFn fn : v.by_kind) {
      const hipError_t e = raise(reinterpret_cast<const void*>(fn));
      if (e != hipSuccess) return static_cast<int>(e);
    }
  for (const StreamVariant& v : kStream) {
    hipError_t e = raise(reinterpret_cast<const void*>(v.fn));
    if (e != hipSuccess) return static_cast<int>(e);
    for (const StreamKernelFn fn : v.by_kind) {
      e = raise(reinterpret_cast<const void*>(fn));
      if (e != hipSuccess) return static_cast<int>(e);
    }
  }
  return static_cast<int>(hipSuccess);
}

// ---- fused: float activations in, q8_1 quantization inside the kernel -------

#define DEFINE_FUSED(QNAME, QT, ANAME, AKIND, ONAME, OKIND)                                              \
  extern "C" int hipengine_gguf_##QNAME##_q8_1_fused_gemv_##ANAME##_##ONAME##_out(                        \
      const void* x, const uint8_t* qweight, void* out, int64_t rows, int64_t in_features,                \
      int64_t out_features, int64_t threads, hipStream_t stream) {                                        \
    (void)threads;                                                                                        \
    return launch_gemv(QT, x, AKIND, qweight, out, OKIND, rows, in_features, out_features, nullptr,       \
                       stream);                                                                           \
  }

#define DEFINE_FUSED_ALL(QNAME, QT)                       \
  DEFINE_FUSED(QNAME, QT, f32, KIND_F32, f32, KIND_F32)   \
  DEFINE_FUSED(QNAME, QT, bf16, KIND_BF16, f32, KIND_F32) \
  DEFINE_FUSED(QNAME, QT, bf16, KIND_BF16, bf16, KIND_BF16) \
  DEFINE_FUSED(QNAME, QT, bf16, KIND_BF16, fp16, KIND_F16) \
  DEFINE_FUSED(QNAME, QT, fp16, KIND_F16, f32, KIND_F32)  \
  DEFINE_FUSED(QNAME, QT, fp16, KIND_F16, fp16, KIND_F16)

DEFINE_FUSED_ALL(q4_k, GGML_Q4_K)
DEFINE_FUSED_ALL(q5_k, GGML_Q5_K)
DEFINE_FUSED_ALL(q6_k, GGML_Q6_K)
DEFINE_FUSED_ALL(q8_0, GGML_Q8_0)

// ---- pre-quantized q8_1 activations (36-byte blocks) ------------------------

#define DEFINE_Q8_1(SYMBOL, QT, OKIND)                                                                   \
  extern "C" int SYMBOL(const void* xq, const uint8_t* qweight, void* out, int64_t rows,                 \
                        int64_t in_features, int64_t out_features, hipStream_t stream) {                 \
    return launch_gemv(QT, xq, KIND_Q8_1, qweight, out, OKIND, rows, in_features, out_features, nullptr, \
                       stream);                                                                          \
  }

DEFINE_Q8_1(hipengine_gguf_q4_k_q8_1_dp4a_vdr_bf16_f32_out, GGML_Q4_K, KIND_F32)
DEFINE_Q8_1(hipengine_gguf_q4_k_q8_1_dp4a_vdr_bf16_bf16_out, GGML_Q4_K, KIND_BF16)
DEFINE_Q8_1(hipengine_gguf_q6_k_q8_1_dp4a_gemv_bf16_f32_out, GGML_Q6_K, KIND_F32)
DEFINE_Q8_1(hipengine_gguf_q6_k_q8_1_dp4a_gemv_bf16_bf16_out, GGML_Q6_K, KIND_BF16)
DEFINE_Q8_1(hipengine_gguf_q8_0_dp4a_gemv_f32_f32_out, GGML_Q8_0, KIND_F32)
DEFINE_Q8_1(hipengine_gguf_q8_0_dp4a_gemv_bf16_bf16_out, GGML_Q8_0, KIND_BF16)

// ---- explicit layout, for tuning sweeps --------------------------------------

extern "C" int hipengine_gfx950_gguf_q8_1_fused_gemv_tuned(
    int32_t ggml_type, const void* x, int32_t x_kind, const uint8_t* qweight, void* out, int32_t out_kind,
    int64_t rows, int64_t in_features, int64_t out_features, int32_t k_slices, int32_t row_groups,
    int32_t blocks_per_wave, int32_t rows_per_lane, hipStream_t stream) {
  if (x_kind < KIND_F32 || x_kind > KIND_Q8_1 || out_kind < KIND_F32 || out_kind > KIND_F16 || rows > 8) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  Plan p;
  p.b = 0;
  p.r = rows_per_lane;
  p.cb = blocks_per_wave;
  p.ks = k_slices;
  p.nrg = row_groups;
  return launch_gemv(ggml_type, x, x_kind, qweight, out, out_kind, rows, in_features, out_features, &p, stream);
}

extern "C" int hipengine_gfx950_gguf_gemv_default_plan(int32_t ggml_type, int64_t rows, int64_t in_features,
                                                       int64_t out_features, int32_t* plan5) {
  if (!plan5 || rows <= 0 || in_features <= 0 || (in_features % QK_K) != 0 || out_features <= 0 ||
      !find_variant(ggml_type, 1, 1, 1)) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  const Plan p = default_plan(ggml_type, static_cast<int>(rows < 8 ? rows : 8), in_features, out_features);
  plan5[0] = p.b; plan5[1] = p.r; plan5[2] = p.cb; plan5[3] = p.ks; plan5[4] = p.nrg;
  return static_cast<int>(hipSuccess);
}

extern "C" int hipengine_gfx950_gguf_gemv_default_form(int32_t ggml_type, int64_t rows, int64_t in_features,
                                                       int64_t out_features, int32_t* form2) {
  if (!form2 || rows <= 0 || in_features <= 0 || (in_features % QK_K) != 0 || out_features <= 0 ||
      !find_variant(ggml_type, 1, 1, 1)) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  int chunk = static_cast<int>(rows < 8 ? rows : 8);
  form2[0] = static_cast<int32_t>(pick_form(ggml_type, chunk, in_features, out_features, nullptr));
  form2[1] = chunk;
  return static_cast<int>(hipSuccess);
}

extern "C" int hipengine_gfx950_gguf_q8_1_fused_gemv_run_tuned(
    int32_t ggml_type, const void* x, int32_t x_kind, const uint8_t* qweight, void* out, int32_t out_kind,
    int64_t rows, int64_t in_features, int64_t out_features, int32_t rows_per_wave, int32_t loads_per_chunk,
    int32_t waves, hipStream_t stream) {
  if (!x || !qweight || !out || x_kind < KIND_F32 || x_kind > KIND_Q8_1 || out_kind < KIND_F32 ||
      out_kind > KIND_F16 || rows <= 0 || rows > 2 || in_features <= 0 || (in_features % QK_K) != 0 ||
      out_features <= 0) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  RunPlan p{};
  p.b = rows <= 1 ? 1 : 2;
  p.g = rows_per_wave;
  p.cb = loads_per_chunk;
  p.waves = waves;
  return launch_gemv_run(ggml_type, x, x_kind, qweight, out, out_kind, static_cast<int>(rows), in_features,
                         out_features, p, stream);
}

extern "C" int hipengine_gfx950_gguf_q8_1_fused_gemv_stream_tuned(
    int32_t ggml_type, const void* x, int32_t x_kind, const uint8_t* qweight, void* out, int32_t out_kind,
    int64_t rows, int64_t in_features, int64_t out_features, int32_t loads_in_flight, int32_t waves,
    int32_t waves_total, hipStream_t stream) {
  if (!x || !qweight || !out || x_kind < KIND_F32 || x_kind > KIND_Q8_1 || out_kind < KIND_F32 ||
      out_kind > KIND_F16 || rows <= 0 || rows > 8 || in_features <= 0 || (in_features % QK_K) != 0 ||
      out_features <= 0) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  StreamPlan p{};
  p.b = batch_bucket(static_cast<int>(rows));
  p.d = loads_in_flight;
  p.waves = waves;
  p.waves_total = waves_total;
  return launch_gemv_stream(ggml_type, x, x_kind, qweight, out, out_kind, static_cast<int>(rows), in_features,
                            out_features, p, stream);
}

extern "C" int hipengine_gfx950_gguf_q4_k_q8_1_fused_gemv_slab_tuned(const void* x, int32_t x_kind,
                                                                    const uint8_t* qweight, void* out,
                                                                    int32_t out_kind, int64_t rows,
                                                                    int64_t in_features, int64_t out_features,
                                                                    int32_t rows_per_workgroup, hipStream_t stream) {
  if (!x || !qweight || !out || x_kind < KIND_F32 || x_kind > KIND_Q8_1 || out_kind < KIND_F32 ||
      out_kind > KIND_F16 || rows <= 0 || rows > 8 || in_features <= 0 || (in_features % QK_K) != 0 ||
      out_features <= 0) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  SlabPlan p = default_slab_plan(GGML_Q4_K, static_cast<int>(rows), in_features, out_features);
  if (!p.ok) return static_cast<int>(hipErrorInvalidValue);
  if (rows_per_workgroup > 0) p.rows_wg = rows_per_workgroup;
  return launch_gemv_slab(x, x_kind, qweight, out, out_kind, static_cast<int>(rows), in_features, out_features, p,
                          stream);
}

extern "C" int hipengine_gfx950_gguf_q8_1_fused_gemv_pslab_tuned(int32_t ggml_type, const void* x, int32_t x_kind,
                                                                const uint8_t* qweight, void* out, int32_t out_kind,
                                                                int64_t rows, int64_t in_features,
                                                                int64_t out_features, int32_t waves,
                                                                int32_t blocks_per_wave, int32_t workgroups,
                                                                hipStream_t stream) {
  if (!x || !qweight || !out || x_kind < KIND_F32 || x_kind > KIND_Q8_1 || out_kind < KIND_F32 ||
      out_kind > KIND_F16 || rows <= 0 || rows > 8 || in_features <= 0 || (in_features % QK_K) != 0 ||
      out_features <= 0) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  PslabPlan p = default_pslab_plan(ggml_type, static_cast<int>(rows), in_features, out_features, qweight);
  if (!p.ok) return static_cast<int>(hipErrorInvalidValue);
  if (waves > 0 || blocks_per_wave > 0) {
    const int nb = static_cast<int>(in_features / QK_K);
    if (waves > 0) p.waves = waves;
    if (blocks_per_wave > 0) p.bpw_log2 = blocks_per_wave == 1 ? 0 : blocks_per_wave == 2 ? 1 : blocks_per_wave == 4 ? 2 : -1;
    if (p.bpw_log2 < 0 || p.waves > 12) return static_cast<int>(hipErrorInvalidValue);
    p.phases = (nb + p.waves * (1 << p.bpw_log2) - 1) / (p.waves * (1 << p.bpw_log2));
    p.grid = pslab_grid(out_features, p.phases);
  }
  if (workgroups > 0) p.grid = workgroups;
  return launch_gemv_pslab(ggml_type, x, x_kind, qweight, out, out_kind, static_cast<int>(rows), in_features,
                           out_features, p, stream);
}

// ---- fused epilogues: gate/up pair with SiLU, projection + residual -------------------

extern "C" int hipengine_gfx950_gguf_pair_silu_gemv(int32_t ggml_type, const void* x, int32_t x_kind,
                                                    const uint8_t* qweight_gate, const uint8_t* qweight_up, void* out,
                                                    int32_t out_kind, int64_t rows, int64_t in_features,
                                                    int64_t out_features, int32_t round_mid, hipStream_t stream) {
  if (!x || !qweight_gate || !qweight_up || !out || x_kind < KIND_F32 || x_kind > KIND_Q8_1 || out_kind < KIND_F32 ||
      out_kind > KIND_F16 || rows <= 0 || rows > 8 || in_features <= 0 || (in_features % QK_K) != 0 ||
      out_features <= 0) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  if (rows > 2) {
    // batch 3..8, on the MFMA forms: the gate projection goes to `out` (rounded to the output type by the
    // store), the up projection's epilogue reads it back: out = silu(gate) * round(up).  That is the
    // round_mid arithmetic, so a 16-bit output without round_mid is not taken.
    if (!round_mid && out_kind != KIND_F32) return static_cast<int>(hipErrorInvalidValue);
    const int r = static_cast<int>(rows);
    const SlabPlan sl = default_slab_plan(ggml_type, r, in_features, out_features);
    if (sl.ok) {
      const int rc = launch_gemv_slab(x, x_kind, qweight_gate, out, out_kind, r, in_features, out_features, sl, stream);
      if (rc != static_cast<int>(hipSuccess)) return rc;
      return launch_gemv_slab(x, x_kind, qweight_up, out, out_kind, r, in_features, out_features, sl, stream, nullptr, out);
    }
    const PslabPlan pg = default_pslab_plan(ggml_type, r, in_features, out_features, qweight_gate);
    const PslabPlan pu = default_pslab_plan(ggml_type, r, in_features, out_features, qweight_up);
    if (!pg.ok || !pu.ok) return static_cast<int>(hipErrorInvalidValue);
    const int rc = launch_gemv_pslab(ggml_type, x, x_kind, qweight_gate, out, out_kind, r, in_features, out_features, pg,
                                     stream);
    if (rc != static_cast<int>(hipSuccess)) return rc;
    return launch_gemv_pslab(ggml_type, x, x_kind, qweight_up, out, out_kind, r, in_features, out_features, pu, stream,
                             nullptr, out);
  }
  const StreamPlan sp = tuned_stream_plan(ggml_type, static_cast<int>(rows), in_features, out_features);
  if (!sp.ok) return static_cast<int>(hipErrorInvalidValue);
  StreamFusion f;
  f.fuse = FUSE_PAIR; f.w_up = qweight_up; f.round_mid = round_mid;
  return launch_gemv_stream(ggml_type, x, x_kind, qweight_gate, out, out_kind, static_cast<int>(rows), in_features,
                            out_features, sp, stream, f);
}

extern "C" int hipengine_gfx950_gguf_gemv_residual(int32_t ggml_type, const void* x, int32_t x_kind,
                                                   const uint8_t* qweight, const void* residual, void* out,
                                                   int32_t out_kind, int64_t rows, int64_t in_features,
                                                   int64_t out_features, hipStream_t stream) {
  if (!x || !qweight || !residual || !out || x_kind < KIND_F32 || x_kind > KIND_Q8_1 || out_kind < KIND_F32 ||
      out_kind > KIND_F16 || rows <= 0 || rows > 8 || in_features <= 0 || (in_features % QK_K) != 0 ||
      out_features <= 0) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  const SlabPlan sl = default_slab_plan(ggml_type, static_cast<int>(rows), in_features, out_features);
  if (slab_preferred(ggml_type, static_cast<int>(rows), in_features, out_features, sl)) {
    return launch_gemv_slab(x, x_kind, qweight, out, out_kind, static_cast<int>(rows), in_features, out_features, sl,
                            stream, residual);
  }
  if (rows > 2) {
    const PslabPlan pp = default_pslab_plan(ggml_type, static_cast<int>(rows), in_features, out_features, qweight);
    if (!pp.ok) return static_cast<int>(hipErrorInvalidValue);
    return launch_gemv_pslab(ggml_type, x, x_kind, qweight, out, out_kind, static_cast<int>(rows), in_features,
                             out_features, pp, stream, residual);
  }
  const StreamPlan sp = tuned_stream_plan(ggml_type, static_cast<int>(rows), in_features, out_features);
  if (!sp.ok) return static_cast<int>(hipErrorInvalidValue);
  StreamFusion f;
  f.fuse = FUSE_RESIDUAL; f.residual = residual;
  return launch_gemv_stream(ggml_type, x, x_kind, qweight, out, out_kind, static_cast<int>(rows), in_features,
                            out_features, sp, stream, f);
}
