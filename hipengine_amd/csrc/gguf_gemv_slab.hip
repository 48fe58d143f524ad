// Slab form of the decode GEMV (Q4_K on the int8 MFMA, one workgroup per CU, waves split K): kernel
// instantiations, planner and launcher.  The kernel body is gguf_gemv_slab.hpp.

#include "gguf_gemv_slab.hpp"
#include "gguf_gemv_launch.hpp"
#include "gguf_init.hpp"

namespace hipengine_gfx950 {

static_assert(SLAB_PAIR_ROWS == SLAB_MAX_PAIR_ROWS, "launcher and kernel agree on the pair limit");

namespace {
// ---- slab form (Q4_K on the int8 MFMA, one workgroup per CU, waves split K) ----

// BPW = 1: up to 16 waves (K <= 4096); BPW = 2: up to 12 waves (K <= 6144), whose 64
// operand registers want the 170-register budget of a 768-thread bound.
template <int B, int BPW, int XK>
__global__ void __launch_bounds__(BPW == 1 ? 1024 : 768) gemv_slab_q4k_kernel(GemvSlabArgs a) {
  extern __shared__ __align__(16) uint8_t smem[];
  gemv_slab_q4k_workgroup<B, BPW, XK>(a, smem, blockIdx.x);
}

// several matrices over one activation (q | k, k | v, ...): every workgroup runs the single-matrix body on its matrix
template <int B, int BPW, int XK>
__global__ void __launch_bounds__(BPW == 1 ? 1024 : 768) gemv_slab_q4k_multi_kernel(GemvSlabMultiArgs m) {
  extern __shared__ __align__(16) uint8_t smem[];
  const int wg = blockIdx.x;
  int i = 0;
  while (i + 1 < m.count && wg >= m.wg_end[i]) ++i;
  gemv_slab_q4k_workgroup<B, BPW, XK>(m.sub[i], smem, wg - (i ? m.wg_end[i - 1] : 0));
}

// gate and up in one launch: out = silu(round(gate.x)) * round(up.x)
template <int B, int BPW, int XK>
__global__ void __launch_bounds__(BPW == 1 ? 1024 : 768) gemv_slab_q4k_pair_kernel(GemvSlabArgs a) {
  extern __shared__ __align__(16) uint8_t smem[];
  gemv_slab_q4k_workgroup<B, BPW, XK, false, true>(a, smem, blockIdx.x);
}

template <int B, int BPW>
__global__ void __launch_bounds__(BPW == 1 ? 1024 : 768) gemv_slab_q4k_dump_kernel(GemvSlabArgs a) {
  extern __shared__ __align__(16) uint8_t smem[];
  gemv_slab_q4k_workgroup<B, BPW, KIND_Q8_1, true>(a, smem, blockIdx.x);
}

using SlabKernelFn = void (*)(GemvSlabArgs);
using SlabMultiKernelFn = void (*)(GemvSlabMultiArgs);
struct SlabVariant {
  int b, bpw;
  SlabKernelFn by_kind[4];
  SlabKernelFn pair_by_kind[4];         // batch buckets 4 and 8 (batch 1 and 2 pair on the stream form)
  SlabMultiKernelFn multi_by_kind[4];   // batch buckets 4 and 8 (batch 1 and 2 share a launch of the stream form)
};
#define SLAB_KINDS(KERNEL, B, BPW) \
  {KERNEL<B, BPW, KIND_F32>, KERNEL<B, BPW, KIND_BF16>, KERNEL<B, BPW, KIND_F16>, KERNEL<B, BPW, KIND_Q8_1>}
#define SLAB_VARIANT(B, BPW)                                                                             \
  SlabVariant { B, BPW, SLAB_KINDS(gemv_slab_q4k_kernel, B, BPW), {nullptr, nullptr, nullptr, nullptr}, \
                {nullptr, nullptr, nullptr, nullptr} }
#define SLAB_VARIANT_PAIR(B, BPW)                                                                               \
  SlabVariant { B, BPW, SLAB_KINDS(gemv_slab_q4k_kernel, B, BPW), SLAB_KINDS(gemv_slab_q4k_pair_kernel, B, BPW), \
                SLAB_KINDS(gemv_slab_q4k_multi_kernel, B, BPW) }
const SlabVariant kSlab[] = {SLAB_VARIANT(1, 1), SLAB_VARIANT(1, 2), SLAB_VARIANT(2, 1), SLAB_VARIANT(2, 2),
                             SLAB_VARIANT_PAIR(4, 1), SLAB_VARIANT_PAIR(4, 2), SLAB_VARIANT_PAIR(8, 1),
                             SLAB_VARIANT_PAIR(8, 2)};




}  // namespace

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
                     int64_t N, const SlabPlan& p, hipStream_t stream, const void* residual,
                     const void* gate, int32_t* dots_out, const uint8_t* w_up) {
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
  // the pair kernels keep 2 x rows_wg partial sums per batch row, and take no other epilogue
  if (w_up && (p.rows_wg > SLAB_MAX_PAIR_ROWS || residual || gate || dots_out || !v->pair_by_kind[x_kind])) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  GemvSlabArgs a{x, w, out, x_kind, out_kind, rows, static_cast<int>(K), static_cast<int>(N), p.rows_wg, p.waves,
                 p.two_block_waves, residual, gate, w_up, dots_out};
  const unsigned grid = static_cast<unsigned>((N + p.rows_wg - 1) / p.rows_wg);
  SlabKernelFn fn = w_up ? v->pair_by_kind[x_kind] : v->by_kind[x_kind];
  if (dots_out) {   // verification: q8_1 activations, batch bucket 8, either block count
    if (x_kind != KIND_Q8_1 || p.b != 8) return static_cast<int>(hipErrorInvalidValue);
    fn = p.bpw == 1 ? gemv_slab_q4k_dump_kernel<8, 1> : gemv_slab_q4k_dump_kernel<8, 2>;
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize,
                                             static_cast<int>(kMaxLds));
    if (e != hipSuccess) return static_cast<int>(e);
  }
  hipLaunchKernelGGL(fn, dim3(grid), dim3(p.waves * 64), lds, stream, a);
  return static_cast<int>(hipGetLastError());
}


// Up to four Q4_K matrices over one activation (batch 3..8) in one launch: the 256 workgroups are shared out in
// proportion to the matrices' rows, every matrix with its own rows per workgroup.
bool slab_multi_ok(int count, const int* qt, int rows, int64_t K, const int64_t* N) {
  if (count < 2 || count > SLAB_MAX_MATRICES || rows < 3 || rows > 8) return false;
  int64_t total = 0;
  for (int i = 0; i < count; ++i) {
    if (qt[i] != GGML_Q4_K || !default_slab_plan(qt[i], rows, K, N[i]).ok) return false;
    total += N[i];
  }
  // every matrix needs a workgroup, and no workgroup more than SLAB_MAX_ROWS rows (checked again by the launcher)
  return total <= static_cast<int64_t>(SLAB_MAX_ROWS) * (kComputeUnits - count);
}

int launch_gemv_slab_multi(int count, const void* x, int x_kind, const uint8_t* const* w, void* const* out, int out_kind,
                           int rows, int64_t K, const int64_t* N, hipStream_t stream) {
  if (count < 2 || count > SLAB_MAX_MATRICES || x_kind < KIND_F32 || x_kind > KIND_Q8_1) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  const SlabPlan p = default_slab_plan(GGML_Q4_K, rows, K, N[0]);
  const SlabVariant* v = nullptr;
  for (const SlabVariant& c : kSlab)
    if (c.b == p.b && c.bpw == p.bpw) v = &c;
  if (!p.ok || !v || !v->multi_by_kind[x_kind]) return static_cast<int>(hipErrorInvalidValue);
  int64_t total = 0;
  for (int i = 0; i < count; ++i) total += N[i];
  GemvSlabMultiArgs m;
  m.count = count;
  int used = 0;
  for (int i = 0; i < count; ++i) {
    // a share of the CUs in proportion to the rows, at least one workgroup; the rows per workgroup follow
    int64_t share = N[i] * kComputeUnits / total;      // rounded down: the shares stay within one round of workgroups
    if (share < 1) share = 1;
    int64_t rows_wg = (N[i] + share - 1) / share;
    if (rows_wg > SLAB_MAX_ROWS) rows_wg = SLAB_MAX_ROWS;
    const int64_t wgs = (N[i] + rows_wg - 1) / rows_wg;
    if (!w[i] || !out[i] || N[i] <= 0 || N[i] > (1 << 30) || used + wgs > (1 << 20)) {
      return static_cast<int>(hipErrorInvalidValue);
    }
    m.sub[i] = GemvSlabArgs{x, w[i], out[i], x_kind, out_kind, rows, static_cast<int>(K), static_cast<int>(N[i]),
                            static_cast<int>(rows_wg), p.waves, p.two_block_waves, nullptr, nullptr, nullptr, nullptr};
    used += static_cast<int>(wgs);
    m.wg_end[i] = used;
  }
  for (int i = count; i < SLAB_MAX_MATRICES; ++i) { m.sub[i] = m.sub[0]; m.wg_end[i] = used; }
  const size_t lds = gemv_slab_lds_bytes(p.b, p.waves, p.two_block_waves);
  if (lds > 160 * 1024) return static_cast<int>(hipErrorInvalidValue);
  if (lds > 64 * 1024) {
    const int rc = ensure_init();
    if (rc != static_cast<int>(hipSuccess)) return rc;
  }
  hipLaunchKernelGGL(v->multi_by_kind[x_kind], dim3(static_cast<unsigned>(used)), dim3(p.waves * 64), lds, stream, m);
  return static_cast<int>(hipGetLastError());
}

int slab_raise_lds_limits() {
  for (const SlabVariant& v : kSlab)
    for (const auto& fns : {v.by_kind, v.pair_by_kind})
      for (int kind = 0; kind < 4; ++kind) {
        if (!fns[kind]) continue;
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(fns[kind]),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(kMaxLds));
        if (e != hipSuccess) return static_cast<int>(e);
      }
  for (const SlabVariant& v : kSlab)
    for (const auto fn : v.multi_by_kind) {
      if (!fn) continue;
      const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize,
                                               static_cast<int>(kMaxLds));
      if (e != hipSuccess) return static_cast<int>(e);
    }
  return static_cast<int>(hipSuccess);
}

}  // namespace hipengine_gfx950
