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
  gemv_slab_q4k_workgroup<B, BPW, XK>(a, smem);
}

// gate and up in one launch: out = silu(round(gate.x)) * round(up.x)
template <int B, int BPW, int XK>
__global__ void __launch_bounds__(BPW == 1 ? 1024 : 768) gemv_slab_q4k_pair_kernel(GemvSlabArgs a) {
  extern __shared__ __align__(16) uint8_t smem[];
  gemv_slab_q4k_workgroup<B, BPW, XK, false, true>(a, smem);
}

template <int B, int BPW>
__global__ void __launch_bounds__(BPW == 1 ? 1024 : 768) gemv_slab_q4k_dump_kernel(GemvSlabArgs a) {
  extern __shared__ __align__(16) uint8_t smem[];
  gemv_slab_q4k_workgroup<B, BPW, KIND_Q8_1, true>(a, smem);
}

using SlabKernelFn = void (*)(GemvSlabArgs);
struct SlabVariant {
  int b, bpw;
  SlabKernelFn by_kind[4];
  SlabKernelFn pair_by_kind[4];   // batch buckets 4 and 8 (batch 1 and 2 pair on the stream form)
};
#define SLAB_KINDS(KERNEL, B, BPW) \
  {KERNEL<B, BPW, KIND_F32>, KERNEL<B, BPW, KIND_BF16>, KERNEL<B, BPW, KIND_F16>, KERNEL<B, BPW, KIND_Q8_1>}
#define SLAB_VARIANT(B, BPW) SlabVariant { B, BPW, SLAB_KINDS(gemv_slab_q4k_kernel, B, BPW), {nullptr, nullptr, nullptr, nullptr} }
#define SLAB_VARIANT_PAIR(B, BPW) \
  SlabVariant { B, BPW, SLAB_KINDS(gemv_slab_q4k_kernel, B, BPW), SLAB_KINDS(gemv_slab_q4k_pair_kernel, B, BPW) }
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


int slab_raise_lds_limits() {
  for (const SlabVariant& v : kSlab)
    for (const auto& fns : {v.by_kind, v.pair_by_kind})
      for (int kind = 0; kind < 4; ++kind) {
        if (!fns[kind]) continue;
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(fns[kind]),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(kMaxLds));
        if (e != hipSuccess) return static_cast<int>(e);
      }
  return static_cast<int>(hipSuccess);
}

}  // namespace hipengine_gfx950
