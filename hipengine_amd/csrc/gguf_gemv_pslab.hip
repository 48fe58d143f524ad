// Phased slab form of the decode GEMV (Q4_K / Q5_K / Q6_K / Q8_0 on the int8 MFMA, batch 3..8): kernel
// instantiations, planner and launcher.  The kernel body is gguf_gemv_pslab.hpp.

#include "gguf_gemv_pslab.hpp"
#include "gguf_gemv_launch.hpp"
#include "gguf_init.hpp"

namespace hipengine_gfx950 {

namespace {
// ---- phased slab form (Q6_K / Q8_0, and Q4_K rows too long for the slab form, on the int8 MFMA; batch 3..8) ----

template <int QT, int B, bool PHASED, int XK>
__global__ void __launch_bounds__(768) gemv_pslab_kernel(GemvPslabArgs a) {
  extern __shared__ __align__(16) uint8_t smem[];
  gemv_pslab_workgroup<QT, B, PHASED, XK>(a, smem);
}

template <int QT, bool PHASED>
__global__ void __launch_bounds__(768) gemv_pslab_dump_kernel(GemvPslabArgs a) {
  extern __shared__ __align__(16) uint8_t smem[];
  gemv_pslab_workgroup<QT, 8, PHASED, KIND_Q8_1, true>(a, smem);
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




}  // namespace

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
                      int64_t K, int64_t N, const PslabPlan& p, hipStream_t stream, const void* residual,
                      const void* gate, int32_t* dots_out) {
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
  a.dots_out = dots_out;
  PslabKernelFn fn = v->by_kind[x_kind];
  if (dots_out) {   // verification: q8_1 activations, batch bucket 8
    if (x_kind != KIND_Q8_1 || p.b != 8) return static_cast<int>(hipErrorInvalidValue);
    const bool ph = p.phases > 1;
    fn = qt == GGML_Q4_K   ? (ph ? gemv_pslab_dump_kernel<GGML_Q4_K, true> : gemv_pslab_dump_kernel<GGML_Q4_K, false>)
         : qt == GGML_Q5_K ? (ph ? gemv_pslab_dump_kernel<GGML_Q5_K, true> : gemv_pslab_dump_kernel<GGML_Q5_K, false>)
         : qt == GGML_Q6_K ? (ph ? gemv_pslab_dump_kernel<GGML_Q6_K, true> : gemv_pslab_dump_kernel<GGML_Q6_K, false>)
                           : (ph ? gemv_pslab_dump_kernel<GGML_Q8_0, true> : gemv_pslab_dump_kernel<GGML_Q8_0, false>);
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize,
                                             static_cast<int>(kMaxLds));
    if (e != hipSuccess) return static_cast<int>(e);
  }
  hipLaunchKernelGGL(fn, dim3(static_cast<unsigned>(p.grid)), dim3(p.waves * 64), lds, stream, a);
  return static_cast<int>(hipGetLastError());
}


int pslab_raise_lds_limits() {
  for (const PslabVariant& v : kPslab)
    for (const auto fn : v.by_kind) {
      if (!fn) continue;
      const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize,
                                               static_cast<int>(kMaxLds));
      if (e != hipSuccess) return static_cast<int>(e);
    }
  return static_cast<int>(hipSuccess);
}

}  // namespace hipengine_gfx950
