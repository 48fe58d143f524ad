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

#define STREAM_RING(D)                                                                                              \
    STREAM_VARIANT_BY_KIND(GGML_Q4_K, 1, D, 2, false), STREAM_VARIANT_BY_KIND(GGML_Q4_K, 2, D, 2, false),               \
    STREAM_VARIANT_BY_KIND(GGML_Q6_K, 1, D, 2, false), STREAM_VARIANT_BY_KIND(GGML_Q6_K, 2, D, 2, false),               \
    STREAM_VARIANT_BY_KIND(GGML_Q8_0, 1, D, 2, false), STREAM_VARIANT_BY_KIND(GGML_Q8_0, 2, D, 2, false),               \
    STREAM_VARIANT_BY_KIND(GGML_Q5_K, 1, D, 2, false), STREAM_VARIANT_BY_KIND(GGML_Q5_K, 2, D, 2, false),               \
    STREAM_VARIANT_BY_KIND(GGML_Q5_K, 1, D, 5, true),                                                                   \
    STREAM_VARIANT_BY_KIND(GGML_Q4_K, 1, D, 5, true), STREAM_VARIANT_BY_KIND(GGML_Q6_K, 1, D, 5, true),                 \
    STREAM_VARIANT_BY_KIND(GGML_Q8_0, 1, D, 5, true),                                                                   \
    STREAM_VARIANT_BY_KIND(GGML_Q4_K, 2, D, 5, true), STREAM_VARIANT_BY_KIND(GGML_Q6_K, 2, D, 5, true),                 \
    STREAM_VARIANT(GGML_Q4_K, 4, D), STREAM_VARIANT(GGML_Q4_K, 8, D), STREAM_VARIANT(GGML_Q6_K, 4, D),                  \
    STREAM_VARIANT(GGML_Q6_K, 8, D), STREAM_VARIANT(GGML_Q8_0, 4, D), STREAM_VARIANT(GGML_Q8_0, 8, D),                  \
    /* gate/up pair with SiLU (Q4_K) and projection + residual (Q4_K, Q6_K), batch 1 and 2 */                           \
    STREAM_VARIANT_FUSED_D(GGML_Q4_K, 1, D, 2, false, FUSE_PAIR), STREAM_VARIANT_FUSED_D(GGML_Q4_K, 2, D, 2, false, FUSE_PAIR),         \
    STREAM_VARIANT_FUSED_D(GGML_Q4_K, 1, D, 2, false, FUSE_RESIDUAL), STREAM_VARIANT_FUSED_D(GGML_Q4_K, 2, D, 2, false, FUSE_RESIDUAL), \
    STREAM_VARIANT_FUSED_D(GGML_Q6_K, 1, D, 2, false, FUSE_RESIDUAL), STREAM_VARIANT_FUSED_D(GGML_Q6_K, 2, D, 2, false, FUSE_RESIDUAL), \
    STREAM_VARIANT_FUSED_D(GGML_Q4_K, 1, D, 5, true, FUSE_RESIDUAL), STREAM_VARIANT_FUSED_D(GGML_Q6_K, 1, D, 5, true, FUSE_RESIDUAL)

const StreamVariant kStream[] = {STREAM_RING(2), STREAM_RING(3)};


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

}  // namespace

// Geometry of a stream launch: rows per chunk (as a shift) and chunks of the matrix.
struct StreamGeometry {
  int chunk_shift;
  int64_t nchunks;
};
StreamGeometry stream_geometry(int nb, int64_t N) {
  StreamGeometry g{0, 0};
  while (((nb << g.chunk_shift) & 15) != 0) ++g.chunk_shift;          // rows per chunk: 16 / gcd(nb, 16)
  g.nchunks = (N + (1 << g.chunk_shift) - 1) >> g.chunk_shift;
  return g;
}

// Groups (per matrix) of the workgroup with the most chunks.
int64_t stream_max_groups(int nb, const StreamGeometry& g, int grid) {
  const int64_t chunks = (g.nchunks + grid - 1) / grid;
  return ((chunks << g.chunk_shift) * nb) / 16;
}

// The stream form applies to K >= 4096 (a group of 16 blocks then spans at most two rows) and
// batch <= 8, from one group per CU on.  One workgroup per CU, two loads in flight per wave (three measured
// slower at every shape and batch).  Waves per workgroup: a workgroup works in rounds of `waves` groups, an
// even number of rounds (the ring is unrolled), and a round of fewer than 8 waves is bound by the latency of
// its loads rather than by their number; so the cost of w waves is rounds(w) * max(w, 8), and the wave
// count is 8 unless another is more than 2 % cheaper.  Measured on MI355X at batch 1 (us, best wave count
// against 8 waves): 17408x5120 Q4_K 11.2 (11 waves) / 11.6; 5120x5120 Q4_K 5.80 (7) / 5.86; 5120x17408 Q6_K
// 18.6 (11) / 18.9; 151936x5120 Q6_K 108.6 (8); 6144x5120 Q4_K 5.95 (8; 5 waves, with no idle slot, 6.7).
// The float32 row sums do not depend on the plan: a group's lanes and the order of a row's groups are fixed by
// K alone.
StreamPlan default_stream_plan(int qt, int rows, int64_t K, int64_t N, int fuse) {
  StreamPlan p{};
  const int nb = static_cast<int>(K / QK_K);
  p.b = batch_bucket(rows);
  p.d = 2;
  p.waves = 8;
  p.waves_total = 0;
  if (rows > 8 || nb < 16 || N < 1) return p;
  const StreamGeometry g = stream_geometry(nb, N);
  const int grid = static_cast<int>(g.nchunks < kComputeUnits ? g.nchunks : kComputeUnits);
  const int mats = fuse == FUSE_PAIR ? 2 : 1;
  const int64_t groups = mats * stream_max_groups(nb, g, grid);
  const int max_waves = p.b == 1 ? 12 : 8;
  auto cost = [&](int w) {
    const int64_t rounds = (groups + w - 1) / w;
    return ((rounds + p.d - 1) / p.d * p.d) * (w < 8 ? 8 : w);
  };
  int64_t best = cost(8);
  for (int w = 5; w <= max_waves; ++w) {
    if (cost(w) * 100 < best * 98) { best = cost(w); p.waves = w; }
  }
  p.waves_total = p.waves * grid;
  p.ok = N * nb / 16 >= kComputeUnits &&
         gemv_run_lds_bytes(qt, p.b, static_cast<int>(K)) + static_cast<size_t>(groups) * 2 * p.b * sizeof(float) <= kMaxLds &&
         pick_stream_variant(qt, p.b, p.d, fuse, nb, p.waves) != nullptr;
  return p;
}

int launch_gemv_stream(int qt, const void* x, int x_kind, const uint8_t* w, void* out, int out_kind, int rows,
                       int64_t K, int64_t N, const StreamPlan& p, hipStream_t stream,
                       const StreamFusion& fusion) {
  const int nb = static_cast<int>(K / QK_K);
  const StreamVariant* v = p.waves > 0 ? pick_stream_variant(qt, p.b, p.d, fusion.fuse, nb, p.waves) : nullptr;
  if (!v || nb < 16 || rows > p.b || p.waves < 1 || p.waves > (p.b == 1 ? 12 : 8) || p.waves_total < p.waves ||
      (p.waves_total % p.waves) != 0) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  if (fusion.fuse == FUSE_PAIR && !fusion.w_up) return static_cast<int>(hipErrorInvalidValue);
  if (fusion.fuse == FUSE_RESIDUAL && !fusion.residual) return static_cast<int>(hipErrorInvalidValue);
  const int grid = p.waves_total / p.waves;
  const int mats = fusion.fuse == FUSE_PAIR ? 2 : 1;
  const StreamGeometry geo = stream_geometry(nb, N);
  const int chunk_shift = geo.chunk_shift;
  const int64_t nchunks = geo.nchunks;
  if (grid > nchunks) return static_cast<int>(hipErrorInvalidValue);
  const int base_chunks = static_cast<int>(nchunks / grid);
  int rounds[2];
  int64_t max_groups = 0;
  for (int big = 0; big < 2; ++big) {
    const int64_t groups = mats * (((static_cast<int64_t>(base_chunks + big) << chunk_shift) * nb) / 16);
    rounds[big] = static_cast<int>((groups + p.waves - 1) / p.waves);
    max_groups = groups;
  }
  // the activation image, then two partial sums per group and batch row
  const size_t lds = gemv_run_lds_bytes(qt, p.b, static_cast<int>(K)) + static_cast<size_t>(max_groups) * 2 * p.b * sizeof(float);
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
  a.chunk_shift = chunk_shift;
  a.base_chunks = base_chunks;
  a.extra_chunks = static_cast<int>(nchunks - static_cast<int64_t>(base_chunks) * grid);
  a.rounds[0] = rounds[0]; a.rounds[1] = rounds[1];
  a.inv_nb = 1.0f / static_cast<float>(nb);
  a.w_up = fusion.w_up; a.residual = fusion.residual; a.round_mid = fusion.round_mid;
  hipLaunchKernelGGL(fn, dim3(grid), dim3(p.waves * 64), lds, stream, a);
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
