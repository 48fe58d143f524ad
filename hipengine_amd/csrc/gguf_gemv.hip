// C entry points of the dense q8_1 decode GEMV (Q4_K / Q6_K / Q8_0, batch 1..8)
// and the launch planner that maps a shape to a workgroup layout.
// The kernel body lives in gguf_gemv.hpp.

#include "gguf_gemv.hpp"
#include "gguf_gemv_run.hpp"
#include "gguf_gemv_launch.hpp"
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
enum GemvForm { FORM_ROW_STRIDED = 0, FORM_RUN = 1, FORM_STREAM = 2, FORM_SLAB = 3, FORM_PSLAB = 4, FORM_DSLAB = 5 };

// Q4_K, K <= 6144: the int8 MFMA slab form wins for batches of 3 and more (17408x5120 at batch 3: 17.0 us against
// 23.0 for the stream form), the stream form at batch 1 and 2 wherever it applies (batch 1: 4.5 against 6.3 us
// at 1024x5120, 10.8 against 15.8 at 17408x5120; batch 2: 5.5 against 6.9 and 14.0 against 15.5; within 0.5 us
// of each other at batch 2 for K = 4096, N = 5120..8192).  Measured on MI355X.
bool slab_preferred(int qt, int chunk, int64_t K, int64_t N, const SlabPlan& sl) {
  if (!sl.ok) return false;
  if (chunk >= 3) return true;
  return !default_stream_plan(qt, chunk, K, N).ok;
}

// The direct slab form is taken where it splits K over workgroups (rows too long for the other MFMA forms to
// hold the quantized activations of): batch 3..8 of K >= 8192 or so.  Measured on MI355X, batch 8 / 4:
// Q6_K 5120x17408 27.1 / 26.0 us against 38.0 / 31.9 for the phased slab, Q4_K 5120x17408 23.5 / 22.4 against
// 28.0 / 23.1, Q8_0 5120x17408 32.6 / 31.5 against 36.8 / 30.3; where K fits one part the older forms are as fast
// or faster (all of them are bound by VALU issue there), and at batch 1 and 2 the stream form is.
bool dslab_preferred(int qt, int chunk, int64_t K, int64_t N, const void* w) {
  // K > 6144: more blocks than the waves of one workgroup hold (Q8_0 at K = 5120 would split as well, for LDS
  // room, and measures slower than the phased slab: 17.3 against 14.7 us at 5120x5120, batch 8)
  if (chunk < (qt == GGML_Q8_0 ? 5 : 3) || K <= 6144) return false;
  const DslabPlan dp = default_dslab_plan(qt, chunk, K, N, w);
  // K parts of equal length only (K = 17408 in 4, 12288 and 8192 in 2: what has been run on hardware); a row whose
  // blocks do not divide (K = 11008: 43 blocks) keeps its older form.  The explicit-layout entry takes any split.
  return dp.ok && dp.ksplit > 1 && (K / QK_K) % dp.ksplit == 0;
}

GemvForm pick_form(int qt, int& chunk, int64_t K, int64_t N, const void* w) {
  if (dslab_preferred(qt, chunk, K, N, w)) return FORM_DSLAB;
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

// What the default dispatch does with a batch of `rows` <= 8 rows of a shape: the form, the rows of the first
// launch and that form's plan.  Planning walks variant tables and LDS budgets (about a microsecond of host time);
// a decode loop asks for the same few shapes over and over, so each thread remembers the last ones.
struct Choice {
  int qt, rows, walign;
  int64_t K, N;
  GemvForm form;
  int chunk;
  SlabPlan slab;
  PslabPlan pslab;
  StreamPlan stream;
  RunPlan run;
  DslabPlan dslab;
};

const Choice& choose(int qt, int rows, int64_t K, int64_t N, const void* w) {
  constexpr int kRemembered = 8;
  thread_local Choice memo[kRemembered];
  thread_local int used = 0, next = 0;
  const int walign = static_cast<int>(reinterpret_cast<uintptr_t>(w) & 3u);
  for (int i = 0; i < used; ++i) {
    const Choice& c = memo[i];
    if (c.qt == qt && c.rows == rows && c.K == K && c.N == N && c.walign == walign) return c;
  }
  Choice& c = memo[next];
  next = (next + 1) % kRemembered;
  used = used < kRemembered ? used + 1 : used;
  c = Choice{};
  c.qt = qt; c.rows = rows; c.walign = walign; c.K = K; c.N = N;
  c.chunk = rows;
  c.form = pick_form(qt, c.chunk, K, N, w);
  switch (c.form) {
    case FORM_DSLAB: c.dslab = default_dslab_plan(qt, c.chunk, K, N, w); break;
    case FORM_SLAB: c.slab = default_slab_plan(qt, c.chunk, K, N); break;
    case FORM_PSLAB: c.pslab = default_pslab_plan(qt, c.chunk, K, N, w); break;
    case FORM_STREAM: c.stream = default_stream_plan(qt, c.chunk, K, N); break;
    case FORM_RUN: c.run = default_run_plan(qt, c.chunk, K, N); break;
    default: break;
  }
  return c;
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
    const Choice* ch = forced ? nullptr : &choose(qt, chunk, K, N, w);
    const GemvForm form = forced ? FORM_ROW_STRIDED : ch->form;
    if (ch) chunk = ch->chunk;
    const int64_t next_r0 = r0 + chunk;
    const void* xr = static_cast<const uint8_t*>(x) + r0 * x_row_bytes;
    void* outr = static_cast<uint8_t*>(out) + r0 * N * out_elem;
    if (form != FORM_ROW_STRIDED) {
      int rc;
      if (form == FORM_DSLAB) {
        rc = launch_gemv_dslab(qt, xr, x_kind, w, outr, out_kind, chunk, K, N, ch->dslab, stream);
      } else if (form == FORM_SLAB) {
        rc = launch_gemv_slab(xr, x_kind, w, outr, out_kind, chunk, K, N, ch->slab, stream);
      } else if (form == FORM_PSLAB) {
        rc = launch_gemv_pslab(qt, xr, x_kind, w, outr, out_kind, chunk, K, N, ch->pslab, stream);
      } else if (form == FORM_STREAM) {
        rc = launch_gemv_stream(qt, xr, x_kind, w, outr, out_kind, chunk, K, N, ch->stream, stream);
      } else {
        rc = launch_gemv_run(qt, xr, x_kind, w, outr, out_kind, chunk, K, N, ch->run, stream);
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
  int rc = slab_raise_lds_limits();
  if (rc == static_cast<int>(hipSuccess)) rc = pslab_raise_lds_limits();
  if (rc == static_cast<int>(hipSuccess)) rc = stream_raise_lds_limits();
  if (rc == static_cast<int>(hipSuccess)) {
    int device = -1;
    rc = static_cast<int>(hipGetDevice(&device));
    if (rc == static_cast<int>(hipSuccess)) rc = dslab_setup(device);
  }
  return rc;
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

// ---- hipEngine's dense names --------------------------------------------------
//
// hipengine_gguf_<q>_gemv_<act>_<out>_out is what hipEngine's dense wrappers bind and what its
// dispatcher reaches through the ("linear", quant, "gemv_*" / "prefill_*") registry keys
// (gguf_q4_k_gemv.hip:2483-2611, gguf_k_gemv.hip:5504-5560).  Here they are the fused kernels above:
// the activations are quantized to q8_1 inside the kernel, so results follow the q8_1 arithmetic of
// hipEngine's dp4a kernels, not the float-activation arithmetic of the kernels of the same name there.

// The dispatcher's prefill_* keys reach the same symbols with many rows (one launch of a (out, rows) grid in
// hipEngine, gguf_q4_k_gemv.hip:1468-1493): from 32 rows of bf16 activations on they are packed, a chunk of up to 512
// rows at a time, into a buffer the library holds and go through the int8-MFMA MMQ - the weights are then read once
// per 512 rows instead of once per 8.
#define DEFINE_DENSE(QNAME, QT, ANAME, AKIND, ONAME, OKIND)                                               \
  extern "C" int hipengine_gguf_##QNAME##_gemv_##ANAME##_##ONAME##_out(                                   \
      const void* x, const uint8_t* qweight, void* out, int64_t rows, int64_t in_features,                \
      int64_t out_features, int64_t threads, hipStream_t stream) {                                        \
    (void)threads;                                                                                        \
    if (AKIND == KIND_BF16 && x && qweight && out &&                                                      \
        prefill_library_buffer_takes(QT, rows, in_features, out_features)) {                              \
      return prefill_bf16_library_buffer(QT, x, qweight, out, OKIND, rows, in_features, out_features, stream); \
    }                                                                                                     \
    return launch_gemv(QT, x, AKIND, qweight, out, OKIND, rows, in_features, out_features, nullptr,       \
                       stream);                                                                           \
  }

// Two matrices over one activation (gate and up, or k and v): out_a = W_a x, out_b = W_b x
// (gguf_k_gemv.hip:5546-5560; Q4_K has the form for its pack8 layout only, gguf_q4_k_gemv.hip:2970).
// One launch of the stream form where it applies (rows <= 2) or of the Q4_K slab form (rows 3..8), else one
// launch per matrix.
int launch_dual(int qt, const void* x, int x_kind, const uint8_t* w_a, const uint8_t* w_b, void* out_a, void* out_b,
                int out_kind, int64_t rows, int64_t K, int64_t N, hipStream_t stream) {
  if (!x || !w_a || !w_b || !out_a || !out_b || rows <= 0 || K <= 0 || N <= 0 || (K % QK_K) != 0) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  if (rows <= 2) {
    const StreamPlan sp = default_stream_plan(qt, static_cast<int>(rows), K, N, FUSE_DUAL);
    if (sp.ok) {
      StreamFusion f;
      f.fuse = FUSE_DUAL; f.w_up = w_b; f.out_b = out_b;
      return launch_gemv_stream(qt, x, x_kind, w_a, out_a, out_kind, static_cast<int>(rows), K, N, sp, stream, f);
    }
  }
  if (rows >= 3 && rows <= 8 && qt == GGML_Q4_K) {   // both on the slab form: one launch of it
    int chunk = static_cast<int>(rows);
    const int q2[2] = {qt, qt};
    const int64_t n2[2] = {N, N};
    if (pick_form(qt, chunk, K, N, w_a) == FORM_SLAB && chunk == rows &&
        slab_multi_ok(2, q2, static_cast<int>(rows), K, n2)) {
      const uint8_t* const w2[2] = {w_a, w_b};
      void* const o2[2] = {out_a, out_b};
      return launch_gemv_slab_multi(2, x, x_kind, w2, o2, out_kind, static_cast<int>(rows), K, n2, stream);
    }
  }
  const int rc = launch_gemv(qt, x, x_kind, w_a, out_a, out_kind, rows, K, N, nullptr, stream);
  if (rc != static_cast<int>(hipSuccess)) return rc;
  return launch_gemv(qt, x, x_kind, w_b, out_b, out_kind, rows, K, N, nullptr, stream);
}

#define DEFINE_DENSE_DUAL(QNAME, QT, ANAME, AKIND, ONAME, OKIND)                                          \
  extern "C" int hipengine_gguf_##QNAME##_dual_gemv_##ANAME##_##ONAME##_out(                              \
      const void* x, const uint8_t* qweight_a, const uint8_t* qweight_b, void* out_a, void* out_b,        \
      int64_t rows, int64_t in_features, int64_t out_features, int64_t threads, hipStream_t stream) {     \
    (void)threads;                                                                                        \
    return launch_dual(QT, x, AKIND, qweight_a, qweight_b, out_a, out_b, OKIND, rows, in_features,        \
                       out_features, stream);                                                             \
  }

#define DEFINE_DENSE_ALL(QNAME, QT)                         \
  DEFINE_DENSE(QNAME, QT, f32, KIND_F32, f32, KIND_F32)     \
  DEFINE_DENSE(QNAME, QT, f32, KIND_F32, fp16, KIND_F16)    \
  DEFINE_DENSE(QNAME, QT, fp16, KIND_F16, f32, KIND_F32)    \
  DEFINE_DENSE(QNAME, QT, fp16, KIND_F16, fp16, KIND_F16)   \
  DEFINE_DENSE(QNAME, QT, bf16, KIND_BF16, f32, KIND_F32)   \
  DEFINE_DENSE(QNAME, QT, bf16, KIND_BF16, fp16, KIND_F16)  \
  DEFINE_DENSE(QNAME, QT, bf16, KIND_BF16, bf16, KIND_BF16) \
  DEFINE_DENSE_DUAL(QNAME, QT, f32, KIND_F32, f32, KIND_F32) \
  DEFINE_DENSE_DUAL(QNAME, QT, bf16, KIND_BF16, bf16, KIND_BF16)

// hipEngine's "rowtile" names (batches of 2 to 8 rows that reuse each weight row across the batch,
// gguf_q4_k_gemv.hip:2496-2533, gguf_k_gemv.hip:5600-5617): every batch here does, so they are the same launch.
#define DEFINE_ROWTILE(QNAME, QT, ANAME, AKIND, ONAME, OKIND)                                             \
  extern "C" int hipengine_gguf_##QNAME##_gemv_rowtile_##ANAME##_##ONAME##_out(                           \
      const void* x, const uint8_t* qweight, void* out, int64_t rows, int64_t in_features,                \
      int64_t out_features, int64_t /*threads*/, hipStream_t stream) {                                    \
    return launch_gemv(QT, x, AKIND, qweight, out, OKIND, rows, in_features, out_features, nullptr,       \
                       stream);                                                                           \
  }
#define DEFINE_ROWTILE_ALL(QNAME, QT)                        \
  DEFINE_ROWTILE(QNAME, QT, f32, KIND_F32, f32, KIND_F32)    \
  DEFINE_ROWTILE(QNAME, QT, bf16, KIND_BF16, f32, KIND_F32)  \
  DEFINE_ROWTILE(QNAME, QT, bf16, KIND_BF16, bf16, KIND_BF16)
DEFINE_ROWTILE_ALL(q4_k, GGML_Q4_K)
DEFINE_ROWTILE_ALL(q5_k, GGML_Q5_K)
DEFINE_ROWTILE_ALL(q6_k, GGML_Q6_K)
DEFINE_ROWTILE_ALL(q8_0, GGML_Q8_0)

DEFINE_DENSE_ALL(q4_k, GGML_Q4_K)
DEFINE_DENSE_ALL(q5_k, GGML_Q5_K)
DEFINE_DENSE_ALL(q6_k, GGML_Q6_K)
DEFINE_DENSE_ALL(q8_0, GGML_Q8_0)

// hipEngine's per-shape tuning variants of the dense GEMV for Q5_K / Q6_K / Q8_0 (row batches, column tiles, wave
// layouts, pipelining: gguf_k_gemv.hip:5665-5702,5869-5960,6161-6255): the same 8 arguments and the same product;
// the launcher here picks the kernel form from the shape, so each of them is the dense launch (any shape, where
// hipEngine restricts some of them to the shapes they were tuned for).
#define DEFINE_DENSE_VARIANT(SYMBOL, QT, AKIND, OKIND)                                                    \
  extern "C" int SYMBOL(const void* x, const uint8_t* qweight, void* out, int64_t rows, int64_t in_features, \
                        int64_t out_features, int64_t /*threads*/, hipStream_t stream) {                  \
    return launch_gemv(QT, x, AKIND, qweight, out, OKIND, rows, in_features, out_features, nullptr, stream); \
  }
#define DEFINE_DENSE_VARIANT_BF16(PREFIX, QT)                          \
  DEFINE_DENSE_VARIANT(PREFIX##_bf16_bf16_out, QT, KIND_BF16, KIND_BF16) \
  DEFINE_DENSE_VARIANT(PREFIX##_bf16_f32_out, QT, KIND_BF16, KIND_F32)
DEFINE_DENSE_VARIANT_BF16(hipengine_gguf_q5_k_gemv_rowbatch8, GGML_Q5_K)
DEFINE_DENSE_VARIANT_BF16(hipengine_gguf_q5_k_gemv_rowbatch32, GGML_Q5_K)
DEFINE_DENSE_VARIANT_BF16(hipengine_gguf_q6_k_gemv_rowbatch8, GGML_Q6_K)
DEFINE_DENSE_VARIANT_BF16(hipengine_gguf_q6_k_gemv_rowbatch32, GGML_Q6_K)
DEFINE_DENSE_VARIANT_BF16(hipengine_gguf_q5_k_gemv_coltile2_rowbatch16, GGML_Q5_K)
DEFINE_DENSE_VARIANT_BF16(hipengine_gguf_q5_k_gemv_coltile4_rowbatch8, GGML_Q5_K)
DEFINE_DENSE_VARIANT_BF16(hipengine_gguf_q6_k_gemv_coltile2_rowbatch16, GGML_Q6_K)
DEFINE_DENSE_VARIANT_BF16(hipengine_gguf_q6_k_gemv_coltile4_rowbatch8, GGML_Q6_K)
DEFINE_DENSE_VARIANT_BF16(hipengine_gguf_q5_k_wave32x2_gemv_decode, GGML_Q5_K)
DEFINE_DENSE_VARIANT_BF16(hipengine_gguf_q5_k_wave32x2_fixed_meta_gemv_decode, GGML_Q5_K)
DEFINE_DENSE_VARIANT_BF16(hipengine_gguf_q5_k_wave32x2_swar_pair_fixed_meta_gemv_decode, GGML_Q5_K)
DEFINE_DENSE_VARIANT(hipengine_gguf_q6_k_wave32x2_fixed_meta_gemv_decode_bf16_bf16_out, GGML_Q6_K, KIND_BF16, KIND_BF16)
DEFINE_DENSE_VARIANT(hipengine_gguf_q6_k_gemv_dpp_wave_reduction_coltile4_rowbatch8_bf16_bf16_out, GGML_Q6_K, KIND_BF16, KIND_BF16)
DEFINE_DENSE_VARIANT(hipengine_gguf_q6_k_gemv_dpp_wave_reduction_coltile2_rowbatch16_bf16_f32_out, GGML_Q6_K, KIND_BF16, KIND_F32)
DEFINE_DENSE_VARIANT(hipengine_gguf_q6_k_gemv_dpp_wave_reduction_full_group_compute_coltile4_rowbatch8_bf16_bf16_out, GGML_Q6_K, KIND_BF16, KIND_BF16)
DEFINE_DENSE_VARIANT(hipengine_gguf_q6_k_gemv_dpp_wave_reduction_full_group_compute_coltile2_rowbatch16_bf16_f32_out, GGML_Q6_K, KIND_BF16, KIND_F32)
DEFINE_DENSE_VARIANT(hipengine_gguf_q8_0_gemv_coltile4_rowbatch8_pipelined_f32_f32_out, GGML_Q8_0, KIND_F32, KIND_F32)
DEFINE_DENSE_VARIANT(hipengine_gguf_q8_0_gemv_coltile8_rowbatch4_pipelined_f32_f32_out, GGML_Q8_0, KIND_F32, KIND_F32)
DEFINE_DENSE_VARIANT(hipengine_gguf_q8_0_gemv_coltile8_rowbatch4_wave_scale_f32_f32_out, GGML_Q8_0, KIND_F32, KIND_F32)
DEFINE_DENSE_VARIANT(hipengine_gguf_q8_0_gemv_coltile8_rowbatch4_wave_scale_pipelined_f32_f32_out, GGML_Q8_0, KIND_F32, KIND_F32)
DEFINE_DENSE_VARIANT(hipengine_gguf_q8_0_gemv_coltile8_rowbatch4_wave_scale_pipelined_dpp_f32_f32_out, GGML_Q8_0, KIND_F32, KIND_F32)
DEFINE_DENSE_VARIANT(hipengine_gguf_q8_0_gemv_coltile8_rowbatch4_wave_scale_pipelined_dpp_checked_full_rows_f32_f32_out, GGML_Q8_0, KIND_F32, KIND_F32)

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
DEFINE_Q8_1(hipengine_gguf_q4_k_q8_1_dp4a_ctl_bf16_f32_out, GGML_Q4_K, KIND_F32)
DEFINE_Q8_1(hipengine_gguf_q4_k_q8_1_dp4a_ctl_bf16_bf16_out, GGML_Q4_K, KIND_BF16)

// The Q8_0 entry points carry a `threads` argument before the stream (ignored, as in hipEngine).  The split
// forms take two or three matrices over the same q8_1 activations, each with its own output buffer.
static int launch_q8_0_split(int count, const void* xq, const uint8_t* const* qweights, void* const* outs, int out_kind,
                             int64_t rows, int64_t in_features, const int64_t* out_features, hipStream_t stream) {
  if (!xq || rows <= 0 || in_features <= 0 || (in_features % QK_K) != 0) return static_cast<int>(hipErrorInvalidValue);
  int qt[4];
  for (int i = 0; i < count; ++i) {
    qt[i] = GGML_Q8_0;
    if (!qweights[i] || !outs[i] || out_features[i] <= 0) return static_cast<int>(hipErrorInvalidValue);
  }
  if (rows <= 2 && stream_multi_ok(count, qt, static_cast<int>(rows), in_features, out_features)) {
    return launch_gemv_stream_multi(count, qt, xq, KIND_Q8_1, qweights, outs, out_kind, static_cast<int>(rows),
                                    in_features, out_features, stream);
  }
  for (int i = 0; i < count; ++i) {
    const int rc = launch_gemv(GGML_Q8_0, xq, KIND_Q8_1, qweights[i], outs[i], out_kind, rows, in_features,
                               out_features[i], nullptr, stream);
    if (rc != static_cast<int>(hipSuccess)) return rc;
  }
  return static_cast<int>(hipSuccess);
}

#define DEFINE_Q8_0_DP4A(SUFFIX, OKIND)                                                                             \
  extern "C" int hipengine_gguf_q8_0_dp4a_gemv_##SUFFIX(const void* xq, const uint8_t* qweight, void* out,          \
                                                        int64_t rows, int64_t in_features, int64_t out_features,    \
                                                        int64_t /*threads*/, hipStream_t stream) {                  \
    return launch_gemv(GGML_Q8_0, xq, KIND_Q8_1, qweight, out, OKIND, rows, in_features, out_features, nullptr,     \
                       stream);                                                                                     \
  }                                                                                                                 \
  extern "C" int hipengine_gguf_q8_0_dp4a_rowtile4_gemv_##SUFFIX(const void* xq, const uint8_t* qweight, void* out, \
                                                                 int64_t rows, int64_t in_features,                 \
                                                                 int64_t out_features, int64_t /*threads*/,         \
                                                                 hipStream_t stream) {                              \
    return launch_gemv(GGML_Q8_0, xq, KIND_Q8_1, qweight, out, OKIND, rows, in_features, out_features, nullptr,     \
                       stream);                                                                                     \
  }                                                                                                                 \
  extern "C" int hipengine_gguf_q8_0_dp4a_dual_split_rowtile4_gemv_##SUFFIX(                                        \
      const void* xq, const uint8_t* qweight_a, const uint8_t* qweight_b, void* out_a, void* out_b, int64_t rows,   \
      int64_t in_features, int64_t out_features_a, int64_t out_features_b, int64_t /*threads*/,                     \
      hipStream_t stream) {                                                                                         \
    const uint8_t* const w[2] = {qweight_a, qweight_b};                                                             \
    void* const o[2] = {out_a, out_b};                                                                              \
    const int64_t n[2] = {out_features_a, out_features_b};                                                          \
    return launch_q8_0_split(2, xq, w, o, OKIND, rows, in_features, n, stream);                                     \
  }                                                                                                                 \
  extern "C" int hipengine_gguf_q8_0_dp4a_triple_split_rowtile4_gemv_##SUFFIX(                                      \
      const void* xq, const uint8_t* qweight_a, const uint8_t* qweight_b, const uint8_t* qweight_c, void* out_a,    \
      void* out_b, void* out_c, int64_t rows, int64_t in_features, int64_t out_features_a, int64_t out_features_b,  \
      int64_t out_features_c, int64_t /*threads*/, hipStream_t stream) {                                            \
    const uint8_t* const w[3] = {qweight_a, qweight_b, qweight_c};                                                  \
    void* const o[3] = {out_a, out_b, out_c};                                                                       \
    const int64_t n[3] = {out_features_a, out_features_b, out_features_c};                                          \
    return launch_q8_0_split(3, xq, w, o, OKIND, rows, in_features, n, stream);                                     \
  }

DEFINE_Q8_0_DP4A(f32_f32_out, KIND_F32)
DEFINE_Q8_0_DP4A(bf16_bf16_out, KIND_BF16)

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

extern "C" int hipengine_gfx950_gguf_q8_1_fused_gemv_dslab_tuned(int32_t ggml_type, const void* x, int32_t x_kind,
                                                                const uint8_t* qweight, void* out, int32_t out_kind,
                                                                int64_t rows, int64_t in_features,
                                                                int64_t out_features, int32_t waves, int32_t ring,
                                                                int32_t workgroups, int32_t k_parts, hipStream_t stream) {
  if (!x || !qweight || !out || x_kind < KIND_F32 || x_kind > KIND_Q8_1 || out_kind < KIND_F32 ||
      out_kind > KIND_F16 || rows <= 0 || rows > 8 || in_features <= 0 || (in_features % QK_K) != 0 ||
      out_features <= 0) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  DslabPlan p = k_parts > 0 ? dslab_plan_for(ggml_type, static_cast<int>(rows), in_features, out_features, qweight, k_parts)
                            : default_dslab_plan(ggml_type, static_cast<int>(rows), in_features, out_features, qweight);
  if (!p.ok) return static_cast<int>(hipErrorInvalidValue);
  if (waves > 0) p.waves = waves;
  if (ring > 0) p.ring = ring;
  if (workgroups > 0) p.row_groups = workgroups / p.ksplit > 0 ? workgroups / p.ksplit : 1;
  return launch_gemv_dslab(ggml_type, x, x_kind, qweight, out, out_kind, static_cast<int>(rows), in_features,
                           out_features, p, stream);
}

// ---- verification: the int32 dots of the MFMA forms -------------------------------------

extern "C" int hipengine_gfx950_gguf_gemv_mfma_dots_i32(int32_t ggml_type, int32_t form, const void* xq,
                                                        const uint8_t* qweight, int32_t* dots, float* out,
                                                        int64_t rows, int64_t in_features, int64_t out_features,
                                                        hipStream_t stream) {
  if (!xq || !qweight || !dots || !out || rows <= 0 || rows > 8 || in_features <= 0 || (in_features % QK_K) != 0 ||
      out_features <= 0) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  // the batch bucket of 8 rows, whatever `rows` is: one verification instantiation per kernel
  if (form == FORM_SLAB) {
    const SlabPlan p = default_slab_plan(ggml_type, 8, in_features, out_features);
    if (!p.ok) return static_cast<int>(hipErrorInvalidValue);
    return launch_gemv_slab(xq, KIND_Q8_1, qweight, out, KIND_F32, static_cast<int>(rows), in_features, out_features, p,
                            stream, nullptr, nullptr, dots);
  }
  if (form == FORM_DSLAB) {
    const DslabPlan p = default_dslab_plan(ggml_type, 8, in_features, out_features, qweight);
    if (!p.ok) return static_cast<int>(hipErrorInvalidValue);
    return launch_gemv_dslab(ggml_type, xq, KIND_Q8_1, qweight, out, KIND_F32, static_cast<int>(rows), in_features,
                             out_features, p, stream, nullptr, nullptr, dots);
  }
  if (form == FORM_PSLAB) {
    const PslabPlan p = default_pslab_plan(ggml_type, 8, in_features, out_features, qweight);
    if (!p.ok) return static_cast<int>(hipErrorInvalidValue);
    return launch_gemv_pslab(ggml_type, xq, KIND_Q8_1, qweight, out, KIND_F32, static_cast<int>(rows), in_features,
                             out_features, p, stream, nullptr, nullptr, dots);
  }
  return static_cast<int>(hipErrorInvalidValue);
}

// ---- several matrices over one activation --------------------------------------------

extern "C" int hipengine_gfx950_gguf_multi_gemv(int32_t count, const int32_t* ggml_types, const void* x, int32_t x_kind,
                                                const uint8_t* const* qweights, void* const* outs, int32_t out_kind,
                                                int64_t rows, int64_t in_features, const int64_t* out_features,
                                                hipStream_t stream) {
  if (count < 1 || count > 4 || !ggml_types || !x || !qweights || !outs || !out_features || x_kind < KIND_F32 ||
      x_kind > KIND_Q8_1 || out_kind < KIND_F32 || out_kind > KIND_F16 || rows <= 0 || in_features <= 0 ||
      (in_features % QK_K) != 0) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  int qt[4];
  for (int i = 0; i < count; ++i) {
    qt[i] = ggml_types[i];
    if (!qweights[i] || !outs[i] || out_features[i] <= 0 || !find_variant(qt[i], 1, 1, 1)) {
      return static_cast<int>(hipErrorInvalidValue);
    }
  }
  if (rows <= 2 && stream_multi_ok(count, qt, static_cast<int>(rows), in_features, out_features)) {
    return launch_gemv_stream_multi(count, qt, x, x_kind, qweights, outs, out_kind, static_cast<int>(rows), in_features,
                                    out_features, stream);
  }
  // batch 3..8: the Q4_K matrices that take the slab form share one launch of it, the others go one by one
  bool done[4] = {false, false, false, false};
  if (rows >= 3 && rows <= 8) {
    int sq[4];
    const uint8_t* sw[4];
    void* so[4];
    int64_t sn[4];
    int picked = 0;
    for (int i = 0; i < count; ++i) {
      int chunk = static_cast<int>(rows);
      if (qt[i] == GGML_Q4_K && pick_form(qt[i], chunk, in_features, out_features[i], qweights[i]) == FORM_SLAB &&
          chunk == rows) {
        sq[picked] = qt[i]; sw[picked] = qweights[i]; so[picked] = outs[i]; sn[picked] = out_features[i];
        ++picked;
      }
    }
    if (picked >= 2 && slab_multi_ok(picked, sq, static_cast<int>(rows), in_features, sn)) {
      const int rc = launch_gemv_slab_multi(picked, x, x_kind, sw, so, out_kind, static_cast<int>(rows), in_features, sn,
                                            stream);
      if (rc != static_cast<int>(hipSuccess)) return rc;
      for (int i = 0; i < count; ++i) {
        for (int j = 0; j < picked; ++j) done[i] = done[i] || (so[j] == outs[i]);
      }
    }
  }
  for (int i = 0; i < count; ++i) {
    if (done[i]) continue;
    const int rc = launch_gemv(qt[i], x, x_kind, qweights[i], outs[i], out_kind, rows, in_features, out_features[i],
                               nullptr, stream);
    if (rc != static_cast<int>(hipSuccess)) return rc;
  }
  return static_cast<int>(hipSuccess);
}

// hipEngine's Q5_K pair decode names (two matrices of different heights over one bf16 activation row,
// gguf_k_gemv.hip:6175-6255): the multi-matrix launch above.
#define DEFINE_Q5_K_PAIR(SYMBOL, OKIND)                                                                       \
  extern "C" int SYMBOL(const void* x, const uint8_t* qweight_a, const uint8_t* qweight_b, void* out_a, void* out_b, \
                        int64_t rows, int64_t in_features, int64_t out_features_a, int64_t out_features_b,       \
                        int64_t /*threads*/, hipStream_t stream) {                                             \
    const int32_t types[2] = {GGML_Q5_K, GGML_Q5_K};                                                           \
    const uint8_t* const weights[2] = {qweight_a, qweight_b};                                                  \
    void* const outs[2] = {out_a, out_b};                                                                      \
    const int64_t heights[2] = {out_features_a, out_features_b};                                               \
    return hipengine_gfx950_gguf_multi_gemv(2, types, x, KIND_BF16, weights, outs, OKIND, rows, in_features,   \
                                            heights, stream);                                                  \
  }
DEFINE_Q5_K_PAIR(hipengine_gguf_q5_k_pair_wave32x2_gemv_decode_bf16_f32_out, KIND_F32)
DEFINE_Q5_K_PAIR(hipengine_gguf_q5_k_pair_wave32x2_fixed_meta_gemv_decode_bf16_bf16_out, KIND_BF16)
DEFINE_Q5_K_PAIR(hipengine_gguf_q5_k_pair_wave32x2_fixed_meta_gemv_decode_bf16_f32_out, KIND_F32)
DEFINE_Q5_K_PAIR(hipengine_gguf_q5_k_pair_wave32x2_swar_pair_fixed_meta_gemv_decode_bf16_bf16_out, KIND_BF16)
DEFINE_Q5_K_PAIR(hipengine_gguf_q5_k_pair_wave32x2_swar_pair_fixed_meta_gemv_decode_bf16_f32_out, KIND_F32)

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
    if (dslab_preferred(ggml_type, r, in_features, out_features, qweight_gate) &&
        dslab_preferred(ggml_type, r, in_features, out_features, qweight_up)) {
      const DslabPlan dg = default_dslab_plan(ggml_type, r, in_features, out_features, qweight_gate);
      const int rc = launch_gemv_dslab(ggml_type, x, x_kind, qweight_gate, out, out_kind, r, in_features, out_features, dg, stream);
      if (rc != static_cast<int>(hipSuccess)) return rc;
      return launch_gemv_dslab(ggml_type, x, x_kind, qweight_up, out, out_kind, r, in_features, out_features,
                               default_dslab_plan(ggml_type, r, in_features, out_features, qweight_up), stream, nullptr, out);
    }
    const SlabPlan sl = default_slab_plan(ggml_type, r, in_features, out_features);
    if (sl.ok) {
      // one launch where a workgroup's rows of both matrices fit its partial-sum buffer (up to 72 x 256 rows)
      if (sl.rows_wg <= SLAB_PAIR_ROWS) {
        return launch_gemv_slab(x, x_kind, qweight_gate, out, out_kind, r, in_features, out_features, sl, stream, nullptr,
                                nullptr, nullptr, qweight_up);
      }
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
  const StreamPlan sp = default_stream_plan(ggml_type, static_cast<int>(rows), in_features, out_features, FUSE_PAIR);
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
  if (dslab_preferred(ggml_type, static_cast<int>(rows), in_features, out_features, qweight)) {
    return launch_gemv_dslab(ggml_type, x, x_kind, qweight, out, out_kind, static_cast<int>(rows), in_features, out_features,
                             default_dslab_plan(ggml_type, static_cast<int>(rows), in_features, out_features, qweight), stream,
                             residual);
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
  const StreamPlan sp = default_stream_plan(ggml_type, static_cast<int>(rows), in_features, out_features, FUSE_RESIDUAL);
  if (!sp.ok) return static_cast<int>(hipErrorInvalidValue);
  StreamFusion f;
  f.fuse = FUSE_RESIDUAL; f.residual = residual;
  return launch_gemv_stream(ggml_type, x, x_kind, qweight, out, out_kind, static_cast<int>(rows), in_features,
                            out_features, sp, stream, f);
}
