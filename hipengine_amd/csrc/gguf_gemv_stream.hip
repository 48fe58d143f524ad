// Stream form of the decode GEMV (resident waves, each with a ring of wave-wide loads in flight; the
// headline batch-1 kernel): kernel instantiations, planner and launcher.  The kernel body is
// gguf_gemv_stream.hpp.

#include "gguf_gemv_stream.hpp"
#include "gguf_gemv_launch.hpp"
#include "gguf_init.hpp"

namespace hipengine_gfx950 {

namespace {
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








}  // namespace

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

int launch_gemv_stream(int qt, const void* x, int x_kind, const uint8_t* w, void* out, int out_kind, int rows,
                       int64_t K, int64_t N, const StreamPlan& p, hipStream_t stream,
                       const StreamFusion& fusion) {
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


int stream_raise_lds_limits() {
  for (const StreamVariant& v : kStream) {
    const void* fns[5] = {reinterpret_cast<const void*>(v.fn), reinterpret_cast<const void*>(v.by_kind[0]),
                          reinterpret_cast<const void*>(v.by_kind[1]), reinterpret_cast<const void*>(v.by_kind[2]),
                          reinterpret_cast<const void*>(v.by_kind[3])};
    for (const void* fn : fns) {
      if (!fn) continue;
      const hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(kMaxLds));
      if (e != hipSuccess) return static_cast<int>(e);
    }
  }
  return static_cast<int>(hipSuccess);
}

}  // namespace hipengine_gfx950
