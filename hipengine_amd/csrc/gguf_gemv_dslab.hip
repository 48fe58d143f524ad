// Direct slab form of the decode GEMV (weights streamed straight into LDS, int8 MFMA, batch 1..8): kernel
// instantiations, planner and launcher.  The kernel body is gguf_gemv_dslab.hpp.

#include "gguf_gemv_dslab.hpp"
#include "gguf_gemv_launch.hpp"
#include "gguf_init.hpp"

#include <atomic>

namespace hipengine_gfx950 {

namespace {

constexpr int DSLAB_MAXB = 2;       // K blocks per wave, at most
constexpr int DSLAB_MAX_WAVES = 12;

// Split-K scratch of the library: partial sums [region][part][8][N] floats and one arrival counter per row
// group and region, zero between launches.  Launches take the regions in turn, so launches that follow each
// other - on one stream or on several - do not share one; more than DSLAB_REGIONS split-K launches in
// flight at once on one device would.
constexpr int DSLAB_REGIONS = 8;
constexpr int DSLAB_REGION_FLOATS = 1 << 20;          // >= parts x 8 batch rows x N
constexpr int DSLAB_MAX_ROW_GROUPS = 1024;
static __device__ __align__(256) float dslab_partials[DSLAB_REGIONS * DSLAB_REGION_FLOATS];
static __device__ __align__(256) uint32_t dslab_counters[DSLAB_REGIONS * DSLAB_MAX_ROW_GROUPS];
constexpr int kMaxDevices = 64;
float* partials_of[kMaxDevices];
uint32_t* counters_of[kMaxDevices];
std::atomic<unsigned> next_region{0};

template <int QT, int XK>
__global__ void __launch_bounds__(DSLAB_MAX_WAVES * 64) gemv_dslab_kernel(GemvDslabArgs a) {
  extern __shared__ __align__(16) uint8_t smem[];
  gemv_dslab_workgroup<QT, DSLAB_MAXB, XK>(a, smem);
}

template <int QT>
__global__ void __launch_bounds__(DSLAB_MAX_WAVES * 64) gemv_dslab_dump_kernel(GemvDslabArgs a) {
  extern __shared__ __align__(16) uint8_t smem[];
  gemv_dslab_workgroup<QT, DSLAB_MAXB, KIND_Q8_1, true>(a, smem);
}

using DslabKernelFn = void (*)(GemvDslabArgs);
struct DslabVariant {
  int qt;
  DslabKernelFn by_kind[4];
  DslabKernelFn dump;
};
#define DSLAB_VARIANT(QT)                                                                             \
  DslabVariant { QT, {gemv_dslab_kernel<QT, KIND_F32>, gemv_dslab_kernel<QT, KIND_BF16>,              \
                      gemv_dslab_kernel<QT, KIND_F16>, gemv_dslab_kernel<QT, KIND_Q8_1>},             \
                 gemv_dslab_dump_kernel<QT> }
const DslabVariant kDslab[] = {DSLAB_VARIANT(GGML_Q4_K), DSLAB_VARIANT(GGML_Q6_K), DSLAB_VARIANT(GGML_Q8_0)};

const DslabVariant* find_dslab(int qt) {
  for (const DslabVariant& v : kDslab)
    if (v.qt == qt) return &v;
  return nullptr;
}

size_t dslab_lds_bytes(int qt, int blocks_part, int waves, int ring, bool red_dedicated) {
  return qt == GGML_Q4_K   ? gemv_dslab_lds_bytes<GGML_Q4_K>(blocks_part, waves, ring, red_dedicated)
         : qt == GGML_Q6_K ? gemv_dslab_lds_bytes<GGML_Q6_K>(blocks_part, waves, ring, red_dedicated)
                           : gemv_dslab_lds_bytes<GGML_Q8_0>(blocks_part, waves, ring, red_dedicated);
}

int dslab_unit_loads(int qt) {   // loads per unit of a wave that owns DSLAB_MAXB blocks
  const int chunks = qt == GGML_Q4_K ? DsTraits<GGML_Q4_K>::CPR : qt == GGML_Q6_K ? DsTraits<GGML_Q6_K>::CPR : DsTraits<GGML_Q8_0>::CPR;
  const int dwords = qt == GGML_Q8_0 ? DsTraits<GGML_Q8_0>::DPR : 0;
  return (DSLAB_MAXB * DS_STEP * chunks + 63) / 64 + (DSLAB_MAXB * DS_STEP * dwords + 63) / 64;
}

int64_t dslab_row_bytes(int qt, int nb) {
  return static_cast<int64_t>(nb) * (qt == GGML_Q4_K ? Q4_K_BYTES : qt == GGML_Q6_K ? Q6_K_BYTES : 8 * Q8_0_BYTES);
}

// steps per group and whether the partial sums need an array of their own
void dslab_groups(int64_t N, int row_groups, int* group, bool* dedicated) {
  const int64_t rows_wg = (N + row_groups - 1) / row_groups;
  const int steps = static_cast<int>((rows_wg + DS_STEP - 1) / DS_STEP);
  *dedicated = steps > DS_GROUP;
  *group = steps > DS_GROUP ? 3 : steps;
}

}  // namespace

// The plan for a given number of K parts (1, 2, 4), `ok` false when the shape does not fit it.
DslabPlan dslab_plan_for(int qt, int rows, int64_t K, int64_t N, const void* w, int parts) {
  DslabPlan p{};
  const int nb = static_cast<int>(K / QK_K);
  if (!find_dslab(qt) || rows < 1 || rows > 8 || (K % QK_K) != 0 || nb < 2 || (reinterpret_cast<uintptr_t>(w) & 1u) != 0 ||
      N < 1 || N > (1 << 24) || N * dslab_row_bytes(qt, nb) > 0xFFFF0000ll || (parts != 1 && parts != 2 && parts != 4)) {
    return p;
  }
  p.ksplit = parts;
  p.blocks_part = (nb + parts - 1) / parts;
  if (p.blocks_part > DSLAB_MAXB * DSLAB_MAX_WAVES || p.blocks_part * (parts - 1) >= nb) return p;    // every part has blocks
  p.waves = p.blocks_part < DSLAB_MAX_WAVES ? p.blocks_part : DSLAB_MAX_WAVES;
  if (p.waves < 2) return p;
  // one workgroup per CU; with K split, as many more rounds of them as keep a workgroup's rows a single group
  const int64_t per_round = kComputeUnits / parts;
  int64_t groups = per_round;
  if (parts > 1) {
    const int64_t need = (N + DS_STEP * DS_GROUP - 1) / (DS_STEP * DS_GROUP);
    groups = (need + per_round - 1) / per_round * per_round;
  }
  p.row_groups = static_cast<int>(N < groups ? N : groups);
  int group;
  bool dedicated;
  dslab_groups(N, p.row_groups, &group, &dedicated);
  // split K needs the library's scratch to hold the partial sums and a single group of steps per workgroup
  if (parts > 1 && (dedicated || N > DSLAB_REGION_FLOATS / (8 * parts) || p.row_groups > DSLAB_MAX_ROW_GROUPS)) return p;
  const int64_t rows_wg = (N + p.row_groups - 1) / p.row_groups;
  const int steps = static_cast<int>((rows_wg + DS_STEP - 1) / DS_STEP);
  int ring = steps + 1 < 4 ? steps + 1 : 4;      // one slot more than the steps: the last slot is the staging scratch
  while (ring >= 2 && (dslab_lds_bytes(qt, p.blocks_part, p.waves, ring, dedicated) > kMaxLds || (ring - 1) * dslab_unit_loads(qt) > 40)) --ring;
  if (ring < 2) return p;
  p.ring = ring;
  p.ok = true;
  return p;
}

// The fewest K parts that give every wave at most MAXB blocks and the ring at least two slots.
DslabPlan default_dslab_plan(int qt, int rows, int64_t K, int64_t N, const void* w) {
  for (int parts = 1; parts <= 4; parts *= 2) {
    const DslabPlan p = dslab_plan_for(qt, rows, K, N, w, parts);
    if (p.ok) return p;
  }
  return DslabPlan{};
}

int launch_gemv_dslab(int qt, const void* x, int x_kind, const uint8_t* w, void* out, int out_kind, int rows,
                      int64_t K, int64_t N, const DslabPlan& p, hipStream_t stream, const void* residual,
                      const void* gate, int32_t* dots_out) {
  const DslabVariant* v = find_dslab(qt);
  const int nb = static_cast<int>(K / QK_K);
  if (!v || rows < 1 || rows > 8 || x_kind < KIND_F32 || x_kind > KIND_Q8_1 || (K % QK_K) != 0 || p.waves < 2 ||
      p.waves > DSLAB_MAX_WAVES || (p.ksplit != 1 && p.ksplit != 2 && p.ksplit != 4) || p.blocks_part < 1 ||
      p.blocks_part * p.ksplit < nb || p.blocks_part * (p.ksplit - 1) >= nb || p.blocks_part > DSLAB_MAXB * p.waves ||
      p.ring < 2 || p.ring > 8 || (p.ring - 1) * dslab_unit_loads(qt) > 40 || p.row_groups < 1 || p.row_groups > N ||
      (reinterpret_cast<uintptr_t>(w) & 1u) != 0 || N > (1 << 24) || N * dslab_row_bytes(qt, nb) > 0xFFFF0000ll) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  int group;
  bool dedicated;
  dslab_groups(N, p.row_groups, &group, &dedicated);
  if (p.ksplit > 1 && (dedicated || N > DSLAB_REGION_FLOATS / (8 * p.ksplit) || p.row_groups > DSLAB_MAX_ROW_GROUPS)) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  const size_t lds = dslab_lds_bytes(qt, p.blocks_part, p.waves, p.ring, dedicated);
  if (lds > kMaxLds) return static_cast<int>(hipErrorInvalidValue);
  GemvDslabArgs a{};
  if (lds > 64 * 1024 || p.ksplit > 1) {
    const int rc = ensure_init();
    if (rc != static_cast<int>(hipSuccess)) return rc;
  }
  if (p.ksplit > 1) {
    int device = -1;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices || !partials_of[device]) {
      return static_cast<int>(hipErrorInvalidDevice);
    }
    const unsigned region = next_region.fetch_add(1, std::memory_order_relaxed) % DSLAB_REGIONS;
    a.partials = partials_of[device] + static_cast<size_t>(region) * DSLAB_REGION_FLOATS;
    a.counters = counters_of[device] + static_cast<size_t>(region) * DSLAB_MAX_ROW_GROUPS;
  }
  a.x = x; a.w = w; a.out = out; a.residual = residual; a.gate = gate;
  a.x_kind = x_kind; a.out_kind = out_kind; a.rows = rows;
  a.K = static_cast<int>(K); a.N = static_cast<int>(N);
  a.waves = p.waves; a.ring = p.ring;
  a.base_rows = static_cast<int>(N / p.row_groups);
  a.group = group; a.red_dedicated = dedicated ? 1 : 0;
  a.ksplit = p.ksplit; a.blocks_part = p.blocks_part;
  a.dots_out = dots_out;
  DslabKernelFn fn = v->by_kind[x_kind];
  if (dots_out) {
    if (x_kind != KIND_Q8_1) return static_cast<int>(hipErrorInvalidValue);
    fn = v->dump;
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize,
                                             static_cast<int>(kMaxLds));
    if (e != hipSuccess) return static_cast<int>(e);
  }
  hipLaunchKernelGGL(fn, dim3(static_cast<unsigned>(p.row_groups * p.ksplit)), dim3(p.waves * 64), lds, stream, a);
  return static_cast<int>(hipGetLastError());
}

// Per device: the dynamic-LDS limit of every kernel and the addresses of the split-K scratch arrays.
int dslab_setup(int device) {
  for (const DslabVariant& v : kDslab)
    for (const auto fn : v.by_kind) {
      const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize,
                                               static_cast<int>(kMaxLds));
      if (e != hipSuccess) return static_cast<int>(e);
    }
  if (device < 0 || device >= kMaxDevices) return static_cast<int>(hipErrorInvalidDevice);
  void* ptr = nullptr;
  hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(dslab_partials));
  if (e != hipSuccess) return static_cast<int>(e);
  partials_of[device] = static_cast<float*>(ptr);
  e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(dslab_counters));
  if (e != hipSuccess) return static_cast<int>(e);
  counters_of[device] = static_cast<uint32_t*>(ptr);
  return static_cast<int>(hipSuccess);
}

}  // namespace hipengine_gfx950
