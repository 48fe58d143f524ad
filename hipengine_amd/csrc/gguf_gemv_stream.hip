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
  gemv_stream_workgroup<QT, B, D, S, XK, FUSE>(a, smem, blockIdx.x, gridDim.x);
}

// Several matrices of any of the four types over one activation, one launch: the grid is split between the
// matrices in proportion to their bytes, and each share runs the plain stream form of its type on its own
// sub-grid (the same chunks, groups and sums as a launch of its own with that many workgroups).
constexpr int STREAM_MULTI_MAX = 4;
struct GemvStreamMultiArgs {
  GemvStreamArgs sub[STREAM_MULTI_MAX];
  int qt[STREAM_MULTI_MAX];
  int wg_end[STREAM_MULTI_MAX];   // workgroups [wg_end[i-1], wg_end[i]) belong to matrix i
  int count;
};

template <int B, int D, int S>
__global__ void __launch_bounds__((stream_max_threads<2>())) gemv_stream_multi_kernel(GemvStreamMultiArgs m) {
  extern __shared__ __align__(16) uint8_t smem[];
  const int wg = blockIdx.x;
  int i = 0;
  while (i + 1 < m.count && wg >= m.wg_end[i]) ++i;
  const int first = i == 0 ? 0 : m.wg_end[i - 1];
  const GemvStreamArgs& a = m.sub[i];
  switch (m.qt[i]) {
    case GGML_Q4_K: gemv_stream_workgroup<GGML_Q4_K, B, D, S>(a, smem, wg - first, m.wg_end[i] - first); break;
    case GGML_Q5_K: gemv_stream_workgroup<GGML_Q5_K, B, D, S>(a, smem, wg - first, m.wg_end[i] - first); break;
    case GGML_Q6_K: gemv_stream_workgroup<GGML_Q6_K, B, D, S>(a, smem, wg - first, m.wg_end[i] - first); break;
    default: gemv_stream_workgroup<GGML_Q8_0, B, D, S>(a, smem, wg - first, m.wg_end[i] - first); break;
  }
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
    STREAM_VARIANT_FUSED_D(GGML_Q4_K, 1, D, 5, true, FUSE_RESIDUAL), STREAM_VARIANT_FUSED_D(GGML_Q6_K, 1, D, 5, true, FUSE_RESIDUAL),               \
    /* two matrices of one shape, two outputs */                                                                        \
    STREAM_VARIANT_FUSED_D(GGML_Q4_K, 1, D, 2, false, FUSE_DUAL), STREAM_VARIANT_FUSED_D(GGML_Q4_K, 2, D, 2, false, FUSE_DUAL),         \
    STREAM_VARIANT_FUSED_D(GGML_Q5_K, 1, D, 2, false, FUSE_DUAL), STREAM_VARIANT_FUSED_D(GGML_Q5_K, 2, D, 2, false, FUSE_DUAL),         \
    STREAM_VARIANT_FUSED_D(GGML_Q6_K, 1, D, 2, false, FUSE_DUAL), STREAM_VARIANT_FUSED_D(GGML_Q6_K, 2, D, 2, false, FUSE_DUAL),         \
    STREAM_VARIANT_FUSED_D(GGML_Q8_0, 1, D, 2, false, FUSE_DUAL), STREAM_VARIANT_FUSED_D(GGML_Q8_0, 2, D, 2, false, FUSE_DUAL)

const StreamVariant kStream[] = {STREAM_RING(2)};


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
  const int mats = (fuse == FUSE_PAIR || fuse == FUSE_DUAL) ? 2 : 1;
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

// Arguments and LDS bytes of a stream launch of `grid` workgroups of `waves` waves.
int stream_fill_args(int qt, const void* x, int x_kind, const uint8_t* w, void* out, int out_kind, int rows, int b,
                     int64_t K, int64_t N, int waves, int grid, const StreamFusion& fusion, GemvStreamArgs& a,
                     size_t& lds) {
  const int nb = static_cast<int>(K / QK_K);
  if (nb < 16 || rows > b || waves < 1 || grid < 1) return static_cast<int>(hipErrorInvalidValue);
  const bool two = fusion.fuse == FUSE_PAIR || fusion.fuse == FUSE_DUAL;
  if (two && !fusion.w_up) return static_cast<int>(hipErrorInvalidValue);
  if (fusion.fuse == FUSE_DUAL && !fusion.out_b) return static_cast<int>(hipErrorInvalidValue);
  if (fusion.fuse == FUSE_RESIDUAL && !fusion.residual) return static_cast<int>(hipErrorInvalidValue);
  const int mats = two ? 2 : 1;
  const StreamGeometry geo = stream_geometry(nb, N);
  const int chunk_shift = geo.chunk_shift;
  const int64_t nchunks = geo.nchunks;
  if (grid > nchunks) return static_cast<int>(hipErrorInvalidValue);
  const int base_chunks = static_cast<int>(nchunks / grid);
  int rounds[2];
  int64_t max_groups = 0;
  for (int big = 0; big < 2; ++big) {
    const int64_t groups = mats * (((static_cast<int64_t>(base_chunks + big) << chunk_shift) * nb) / 16);
    rounds[big] = static_cast<int>((groups + waves - 1) / waves);
    max_groups = groups;
  }
  // the activation image, then two partial sums per group and batch row
  lds = gemv_run_lds_bytes(qt, b, static_cast<int>(K)) + static_cast<size_t>(max_groups) * 2 * b * sizeof(float);
  if (lds > kMaxLds) return static_cast<int>(hipErrorInvalidValue);
  a.x = x; a.w = w; a.out = out;
  a.x_kind = x_kind; a.out_kind = out_kind;
  a.rows = rows; a.K = static_cast<int>(K); a.N = static_cast<int>(N);
  a.waves = waves; a.waves_total = waves * grid;
  a.chunk_shift = chunk_shift;
  a.base_chunks = base_chunks;
  a.extra_chunks = static_cast<int>(nchunks - static_cast<int64_t>(base_chunks) * grid);
  a.rounds[0] = rounds[0]; a.rounds[1] = rounds[1];
  a.inv_nb = 1.0f / static_cast<float>(nb);
  a.w_up = fusion.w_up; a.residual = fusion.residual; a.round_mid = fusion.round_mid; a.out_b = fusion.out_b;
  return static_cast<int>(hipSuccess);
}

int launch_gemv_stream(int qt, const void* x, int x_kind, const uint8_t* w, void* out, int out_kind, int rows,
                       int64_t K, int64_t N, const StreamPlan& p, hipStream_t stream,
                       const StreamFusion& fusion) {
  const int nb = static_cast<int>(K / QK_K);
  const StreamVariant* v = p.waves > 0 ? pick_stream_variant(qt, p.b, p.d, fusion.fuse, nb, p.waves) : nullptr;
  if (!v || p.waves > (p.b == 1 ? 12 : 8) || p.waves_total < p.waves || (p.waves_total % p.waves) != 0) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  const int grid = p.waves_total / p.waves;
  GemvStreamArgs a;
  size_t lds = 0;
  const int rc = stream_fill_args(qt, x, x_kind, w, out, out_kind, rows, p.b, K, N, p.waves, grid, fusion, a, lds);
  if (rc != static_cast<int>(hipSuccess)) return rc;
  // the kind-specialised kernels stage the whole row from the groups fetched up front
  const bool up_front = nb * 8 <= v->s * p.waves * 16;
  const StreamKernelFn fn =
      (up_front && x_kind >= KIND_F32 && x_kind <= KIND_Q8_1 && v->by_kind[x_kind]) ? v->by_kind[x_kind] : v->fn;
  if (lds > 64 * 1024) {
    const int rc2 = ensure_init();
    if (rc2 != static_cast<int>(hipSuccess)) return rc2;
  }
  hipLaunchKernelGGL(fn, dim3(grid), dim3(p.waves * 64), lds, stream, a);
  return static_cast<int>(hipGetLastError());
}

// Whether `count` matrices of these types and row counts over one activation of K values can go as one launch.
bool stream_multi_ok(int count, const int* qt, int rows, int64_t K, const int64_t* N) {
  if (count < 1 || count > STREAM_MULTI_MAX || rows < 1 || rows > 2 || K < 16 * QK_K || (K % QK_K) != 0) return false;
  int64_t chunks = 0;
  for (int i = 0; i < count; ++i) {
    if (qt[i] != GGML_Q4_K && qt[i] != GGML_Q5_K && qt[i] != GGML_Q6_K && qt[i] != GGML_Q8_0) return false;
    if (N[i] < 1 || N[i] > (1 << 30)) return false;
    chunks += stream_geometry(static_cast<int>(K / QK_K), N[i]).nchunks;
  }
  return chunks >= count;
}

int launch_gemv_stream_multi(int count, const int* qt, const void* x, int x_kind, const uint8_t* const* w,
                             void* const* out, int out_kind, int rows, int64_t K, const int64_t* N,
                             hipStream_t stream) {
  if (!stream_multi_ok(count, qt, rows, K, N)) return static_cast<int>(hipErrorInvalidValue);
  const int nb = static_cast<int>(K / QK_K);
  const int b = batch_bucket(rows), waves = 8;
  // workgroups per matrix in proportion to its bytes, at least one, at most one per chunk
  int64_t bytes[STREAM_MULTI_MAX], chunks[STREAM_MULTI_MAX], total_bytes = 0, total_chunks = 0;
  for (int i = 0; i < count; ++i) {
    const int64_t super = qt[i] == GGML_Q4_K ? Q4_K_BYTES : qt[i] == GGML_Q5_K ? Q5_K_BYTES : qt[i] == GGML_Q6_K ? Q6_K_BYTES : 8 * Q8_0_BYTES;
    bytes[i] = N[i] * nb * super;
    chunks[i] = stream_geometry(nb, N[i]).nchunks;
    total_bytes += bytes[i];
    total_chunks += chunks[i];
  }
  const int grid_total = static_cast<int>(total_chunks < kComputeUnits ? total_chunks : kComputeUnits);
  int share[STREAM_MULTI_MAX], given = 0;
  for (int i = 0; i < count; ++i) {
    int64_t s = (bytes[i] * grid_total + total_bytes / 2) / total_bytes;
    s = s < 1 ? 1 : s > chunks[i] ? chunks[i] : s;
    share[i] = static_cast<int>(s);
    given += share[i];
  }
  // the rounding difference goes, one workgroup at a time, to the matrix with the most bytes per workgroup
  // (or comes from the one with the fewest)
  while (given != grid_total) {
    const bool grow = given < grid_total;
    int best = -1;
    for (int i = 0; i < count; ++i) {
      if (grow ? share[i] >= chunks[i] : share[i] <= 1) continue;
      if (best < 0) { best = i; continue; }
      const bool more = bytes[i] * share[best] > bytes[best] * share[i];   // bytes per workgroup: i against best
      if (more == grow) best = i;
    }
    if (best < 0) break;
    share[best] += grow ? 1 : -1;
    given += grow ? 1 : -1;
  }
  GemvStreamMultiArgs m;
  m.count = count;
  size_t lds = 0;
  int end = 0;
  for (int i = 0; i < STREAM_MULTI_MAX; ++i) {
    const int k = i < count ? i : count - 1;           // unused slots repeat the last matrix
    size_t l = 0;
    const int rc = stream_fill_args(qt[k], x, x_kind, w[k], out[k], out_kind, rows, b, K, N[k], waves, share[k],
                                    StreamFusion{}, m.sub[i], l);
    if (rc != static_cast<int>(hipSuccess)) return rc;
    if (!w[k] || !out[k]) return static_cast<int>(hipErrorInvalidValue);
    lds = l > lds ? l : lds;
    m.qt[i] = qt[k];
    if (i < count) end += share[i];
    m.wg_end[i] = end;
  }
  if (lds > 64 * 1024) {
    const int rc = ensure_init();
    if (rc != static_cast<int>(hipSuccess)) return rc;
  }
  if (b == 1) {
    hipLaunchKernelGGL((gemv_stream_multi_kernel<1, 2, 2>), dim3(end), dim3(waves * 64), lds, stream, m);
  } else {
    hipLaunchKernelGGL((gemv_stream_multi_kernel<2, 2, 2>), dim3(end), dim3(waves * 64), lds, stream, m);
  }
  return static_cast<int>(hipGetLastError());
}

int stream_raise_lds_limits() {
  for (const void* fn : {reinterpret_cast<const void*>(gemv_stream_multi_kernel<1, 2, 2>),
                         reinterpret_cast<const void*>(gemv_stream_multi_kernel<2, 2, 2>)}) {
    const hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(kMaxLds));
    if (e != hipSuccess) return static_cast<int>(e);
  }
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
