/*
 * C ABI of libhipengine_gfx950.so: hand-written gfx950 (MI355X, CDNA4) kernels
 * for hipEngine's GGUF k-quant matmul path.
 *
 * Conventions shared by every entry point (they are hipEngine's own, see
 * kernels/hip_gfx1100/quant/gguf_q4_k_gemv.hip:2483-2611 in the hipEngine tree):
 *   - plain device pointers and int64 sizes; bf16/fp16 travel as uint16 bits;
 *   - the caller owns every buffer; nothing is allocated, copied or synchronized;
 *   - the launch is asynchronous on `stream` (0 = the null stream) and may be
 *     captured into a HIP graph;
 *   - the return value is a hipError_t as int: hipErrorInvalidValue (1) for
 *     rejected arguments, otherwise hipGetLastError() after the launch;
 *   - weights are raw GGUF block bytes, row major [out_features, row_bytes],
 *     expert tensors [experts, out_features, row_bytes];
 *   - `threads` is accepted for signature compatibility and ignored.
 *
 * Names: where an entry point replaces one of hipEngine's, it keeps that name
 * and the comment cites the hipEngine definition (file:line).  Entry points
 * that exist only here are prefixed hipengine_gfx950_ or carry "fused" in the
 * name, and say so.
 */
#ifndef HIPENGINE_GFX950_H
#define HIPENGINE_GFX950_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#ifndef HIPENGINE_GFX950_STREAM_T
#define HIPENGINE_GFX950_STREAM_T
typedef struct ihipStream_t* hipengine_stream_t; /* == hipStream_t */
#endif

/* Element kinds for the entry points that take them as arguments. */
#define HIPENGINE_GFX950_F32 0
#define HIPENGINE_GFX950_BF16 1
#define HIPENGINE_GFX950_F16 2
#define HIPENGINE_GFX950_Q8_1 3

/* ------------------------------------------------------------------------
 * Library
 * ------------------------------------------------------------------------ */

/* ABI revision of this header; bumped on any incompatible change.  New here. */
int hipengine_gfx950_abi_version(void);

/* ------------------------------------------------------------------------
 * q8_1 activation quantizers
 * ------------------------------------------------------------------------ */

/* [rows, in_features] -> 36-byte block_q8_1 {half d; half s; int8 qs[32]} blocks,
 * [rows, in_features/32].  d = amax/127, q = clamp(roundf(x/d), -128, 127),
 * s = sum of the inputs.  in_features % 32 == 0.
 * Replaces gguf_q4_k_gemv.hip:2834-2862 (kernel :740-772). */
int hipengine_gguf_q4_k_quantize_f32_q8_1(const void* x, void* xq, int64_t rows, int64_t in_features,
                                          hipengine_stream_t stream);
int hipengine_gguf_q4_k_quantize_bf16_q8_1(const void* x, void* xq, int64_t rows, int64_t in_features,
                                           hipengine_stream_t stream);

/* bf16 [rows, hidden] -> 144-byte DS4 blocks {half ds4[8]; int8 qs[128]},
 * [rows, hidden/128]: per 32 values scale = min(65504, amax/127),
 * q = clamp(rint(x/scale), -127, 127), ds4[2g] = half(scale), ds4[2g+1] = half(sum).
 * hidden % 128 == 0.
 * Replaces gguf_q4_k_q8_1_selected_prefill.hip:5582-5594 (kernel :627-690). */
int hipengine_gguf_q8_1_mmq_ds4_pack_bf16(const void* x, void* out, int64_t rows, int64_t hidden,
                                          hipengine_stream_t stream);

/* bf16 [rows, hidden] -> 160-byte D4S4 blocks {float d4[4]; float s4[4]; int8 qs[128]}:
 * d = amax/127 (float32), q = clamp(roundf(x/d), -128, 127).  hidden % 128 == 0.
 * Replaces gguf_k_mmq_prefill.hip:2515-2540 (kernel :264-307). */
int hipengine_gguf_q8_1_d4s4_f32_quantize_bf16(const void* x, void* out, int64_t rows, int64_t hidden,
                                               hipengine_stream_t stream);

/* ------------------------------------------------------------------------
 * Decode GEMV, batch 1..8 per launch (more rows are split into launches of 8)
 *   out[r, n] = sum_k W[n, k] * x[r, k],  W raw Q4_K / Q6_K / Q8_0 blocks
 * in_features % 256 == 0 for all three weight types.
 * ------------------------------------------------------------------------ */

/* Fused: x is [rows, in_features] float32 / bf16 / fp16; the q8_1 quantization
 * above happens inside the kernel and the matmul is int8 dots with a float32
 * combine.  Same argument list as hipEngine's float-activation GEMV
 * (gguf_q4_k_gemv.hip:2483-2611), so a wrapper can swap one for the other.
 * New here (hipEngine runs quantize and GEMV as two launches,
 * runtime/gguf_linear.py:7118-7154). */
#define HIPENGINE_GFX950_DECLARE_FUSED(q, a, o)                                                          \
  int hipengine_gguf_##q##_q8_1_fused_gemv_##a##_##o##_out(                                              \
      const void* x, const uint8_t* qweight, void* out, int64_t rows, int64_t in_features,               \
      int64_t out_features, int64_t threads, hipengine_stream_t stream);
#define HIPENGINE_GFX950_DECLARE_FUSED_ALL(q) \
  HIPENGINE_GFX950_DECLARE_FUSED(q, f32, f32) \
  HIPENGINE_GFX950_DECLARE_FUSED(q, bf16, f32) \
  HIPENGINE_GFX950_DECLARE_FUSED(q, bf16, bf16) \
  HIPENGINE_GFX950_DECLARE_FUSED(q, bf16, fp16) \
  HIPENGINE_GFX950_DECLARE_FUSED(q, fp16, f32) \
  HIPENGINE_GFX950_DECLARE_FUSED(q, fp16, fp16)
HIPENGINE_GFX950_DECLARE_FUSED_ALL(q4_k)
HIPENGINE_GFX950_DECLARE_FUSED_ALL(q6_k)
HIPENGINE_GFX950_DECLARE_FUSED_ALL(q8_0)

/* Pre-quantized: xq is [rows, in_features/32] 36-byte q8_1 blocks.
 * Q4_K replaces gguf_q4_k_q8_1_dp4a_vdr_gemv.hip:321-361 (without its
 * out_features % 8 restriction); Q8_0 replaces gguf_q8_0_dp4a_gemv.hip:345-388;
 * the Q6_K pair is new here (hipEngine has the Q6_K q8_1 dot only in its
 * expert-selected kernel, gguf_k_gemv.hip:3989-4088). */
int hipengine_gguf_q4_k_q8_1_dp4a_vdr_bf16_f32_out(const void* xq, const uint8_t* qweight, void* out, int64_t rows,
                                                   int64_t in_features, int64_t out_features,
                                                   hipengine_stream_t stream);
int hipengine_gguf_q4_k_q8_1_dp4a_vdr_bf16_bf16_out(const void* xq, const uint8_t* qweight, void* out, int64_t rows,
                                                    int64_t in_features, int64_t out_features,
                                                    hipengine_stream_t stream);
int hipengine_gguf_q6_k_q8_1_dp4a_gemv_bf16_f32_out(const void* xq, const uint8_t* qweight, void* out, int64_t rows,
                                                    int64_t in_features, int64_t out_features,
                                                    hipengine_stream_t stream);
int hipengine_gguf_q6_k_q8_1_dp4a_gemv_bf16_bf16_out(const void* xq, const uint8_t* qweight, void* out, int64_t rows,
                                                     int64_t in_features, int64_t out_features,
                                                     hipengine_stream_t stream);
int hipengine_gguf_q8_0_dp4a_gemv_f32_f32_out(const void* xq, const uint8_t* qweight, void* out, int64_t rows,
                                              int64_t in_features, int64_t out_features, hipengine_stream_t stream);
int hipengine_gguf_q8_0_dp4a_gemv_bf16_bf16_out(const void* xq, const uint8_t* qweight, void* out, int64_t rows,
                                                int64_t in_features, int64_t out_features,
                                                hipengine_stream_t stream);

/* The fused GEMV with an explicit workgroup layout, for tuning sweeps: a
 * workgroup is k_slices x row_groups waves, every wave walks blocks_per_wave
 * 256-value blocks per chunk of rows_per_lane x 16 rows.  rows <= 8.  New here. */
int hipengine_gfx950_gguf_q8_1_fused_gemv_tuned(int32_t ggml_type, const void* x, int32_t x_kind,
                                                const uint8_t* qweight, void* out, int32_t out_kind, int64_t rows,
                                                int64_t in_features, int64_t out_features, int32_t k_slices,
                                                int32_t row_groups, int32_t blocks_per_wave, int32_t rows_per_lane,
                                                hipengine_stream_t stream);

/* The same for the "run" form of the kernel (a wave streams rows_per_wave whole
 * rows as one contiguous run of blocks, loads_per_chunk 16-block loads at a
 * time, `waves` waves per workgroup).  rows <= 2, rows_per_wave * (K/256) must
 * be a multiple of 16.  New here. */
int hipengine_gfx950_gguf_q8_1_fused_gemv_run_tuned(int32_t ggml_type, const void* x, int32_t x_kind,
                                                    const uint8_t* qweight, void* out, int32_t out_kind,
                                                    int64_t rows, int64_t in_features, int64_t out_features,
                                                    int32_t rows_per_wave, int32_t loads_per_chunk, int32_t waves,
                                                    hipengine_stream_t stream);

/* The same for the "stream" form (waves_total resident waves, `waves` per
 * workgroup, each owning a contiguous range of rows and keeping loads_in_flight
 * 16-block loads in flight).  rows <= 2, in_features >= 4096,
 * waves_total <= out_features.  New here. */
int hipengine_gfx950_gguf_q8_1_fused_gemv_stream_tuned(int32_t ggml_type, const void* x, int32_t x_kind,
                                                       const uint8_t* qweight, void* out, int32_t out_kind,
                                                       int64_t rows, int64_t in_features, int64_t out_features,
                                                       int32_t loads_in_flight, int32_t waves, int32_t waves_total,
                                                       hipengine_stream_t stream);

/* Host only: the layout the library picks for a shape, as
 * {batch_bucket, rows_per_lane, blocks_per_wave, k_slices, row_groups}.  New here. */
int hipengine_gfx950_gguf_gemv_default_plan(int32_t ggml_type, int64_t rows, int64_t in_features,
                                            int64_t out_features, int32_t* plan5);

/* ------------------------------------------------------------------------
 * MMQ prefill GEMM on int8 MFMA
 *   out[m, n] = sum_k W[n, k] * x[m, k],  x pre-quantized to q8_1 (128-value blocks)
 * rows <= 2^20, in_features % 256 == 0, out_features % 32 == 0.
 * ------------------------------------------------------------------------ */

/* Raw Q4_K weights x DS4 activations ([rows, in_features/128] 144-byte blocks):
 * sum_j (d*sc_j)*xd_j*dot_j - (dmin*mn_j)*xsum_j per 32-wide sub-block.
 * Replaces gguf_q4_k_q8_1_mmq_prefill.hip:421-454,516-519 (kernel :158-289); the
 * ctl and vdr names are the same kernel here, as their results are identical by
 * hipEngine's own contract (:20-27). */
int hipengine_gguf_q4_k_q8_1_mmq32_vdr_dense_bf16_f32_out(const void* xq, const uint8_t* qweight, void* out,
                                                          int64_t rows, int64_t in_features, int64_t out_features,
                                                          hipengine_stream_t stream);
int hipengine_gguf_q4_k_q8_1_mmq32_vdr_dense_bf16_bf16_out(const void* xq, const uint8_t* qweight, void* out,
                                                           int64_t rows, int64_t in_features, int64_t out_features,
                                                           hipengine_stream_t stream);
int hipengine_gguf_q4_k_q8_1_mmq32_ctl_dense_bf16_f32_out(const void* xq, const uint8_t* qweight, void* out,
                                                          int64_t rows, int64_t in_features, int64_t out_features,
                                                          hipengine_stream_t stream);
int hipengine_gguf_q4_k_q8_1_mmq32_ctl_dense_bf16_bf16_out(const void* xq, const uint8_t* qweight, void* out,
                                                           int64_t rows, int64_t in_features, int64_t out_features,
                                                           hipengine_stream_t stream);

/* Raw Q6_K weights x D4S4 activations ([rows, in_features/128] 160-byte blocks
 * {float d4[4]; float s4[4]; int8 qs[128]}): sum over 32-value groups of
 * xd_g * (s0*dot0 + s1*dot1), s = d*scale_i8 per 16 values, dots of the centred
 * 6-bit values.  Any out_features >= 1.
 * Replaces gguf_k_mmq_prefill.hip:2588 (HIPENGINE_GGUF_K_MMQ_EXPORTS(gguf_q6_k, 6);
 * kernel :519-685), Python side gguf_k_mmq_prefill.py:349-397. */
int hipengine_gguf_q6_k_mmq32_q8_1_d4s4_f32_bf16_f32_out(const void* xq, const uint8_t* qweight, void* out,
                                                         int64_t rows, int64_t in_features, int64_t out_features,
                                                         hipengine_stream_t stream);
int hipengine_gguf_q6_k_mmq32_q8_1_d4s4_f32_bf16_bf16_out(const void* xq, const uint8_t* qweight, void* out,
                                                          int64_t rows, int64_t in_features, int64_t out_features,
                                                          hipengine_stream_t stream);

/* The same Q4_K x DS4 GEMM with the kernel form chosen by the caller (benchmarks
 * and tuning; no counterpart in hipEngine).  out_kind: 0 float32, 1 bf16, 2 fp16.
 * variant 0: the next K step is prefetched into registers (what the named entry
 * points run); variant 1: no prefetch, one more workgroup per CU. */
int hipengine_gfx950_gguf_q4_k_mmq_tuned(const void* xq, const uint8_t* qweight, void* out, int out_kind,
                                         int64_t rows, int64_t in_features, int64_t out_features, int variant,
                                         hipengine_stream_t stream);

/* ------------------------------------------------------------------------
 * Verification exports: the integer unpack and the int32 sub-block dots the
 * production kernels compute, written out so that they can be compared bit for
 * bit with a CPU oracle.  New here.
 * ------------------------------------------------------------------------ */

/* n_blocks raw blocks -> float32 values (256 per Q4_K/Q6_K block, 32 per Q8_0
 * block), the arithmetic of hipengine/quant/gguf.py:604-681. */
int hipengine_gfx950_gguf_dequantize_f32(int32_t ggml_type, const uint8_t* blocks, float* out, int64_t n_blocks,
                                         hipengine_stream_t stream);

/* xq: 36-byte q8_1 blocks [rows, K/32].  dots: int32 [rows, out_features, K/32]
 * (Q6_K: K/16, already minus 32*qsum16).  qsums: int32 [rows, K/32] sums of the
 * q8 values (may be NULL). */
int hipengine_gfx950_gguf_q8_1_block_dots_i32(int32_t ggml_type, const void* xq, const uint8_t* qweight,
                                              int32_t* dots, int32_t* qsums, int64_t rows, int64_t in_features,
                                              int64_t out_features, hipengine_stream_t stream);

#ifdef __cplusplus
}
#endif

#endif /* HIPENGINE_GFX950_H */
