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

#include <stdbool.h>
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

/* Per-device set-up, for the device that is current: raises the dynamic-LDS limit of every kernel
 * that may need more than the default 64 KB and looks up the addresses of the device arrays the
 * library holds (the scratch of hipengine_gfx950_argmax_f32_rows_i32_noalloc, the pack buffer of the
 * dense prefill entries, the partial sums of the split-K decode GEMV).  Call it once per device after
 * loading the library and before capturing a HIP graph; after it, no entry point makes any call that
 * is not a stream operation, so every one of them can be captured from its first launch on - except
 * the verification exports (hipengine_gfx950_gguf_gemv_mfma_dots_i32), which set a kernel attribute
 * on every call and are not meant for graphs.  Entry points that need the set-up run it themselves
 * when it has not been done (then outside of a capture, please).
 * Allocates nothing; safe to call again and from several threads.  New here. */
int hipengine_gfx950_init(void);

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

/* bf16 [rows, in_features] -> two planes [2, rows, in_features/32] of block_q8_1: plane 0 is the quantization above,
 * plane 1 (at + rows * in_features/32 blocks) the same quantization of the residual x - float(half d0) * q0.
 * Replaces gguf_q4_k_gemv.hip:2844-2852 (kernel :777-829).  hipEngine's consumers of the two planes take its RDNA3
 * weight layouts; here the planes are 2 * rows rows of the pre-quantized q8_1 GEMV, whose two results add up. */
int hipengine_gguf_q4_k_quantize_bf16_q8_1x2(const void* x, void* xq, int64_t rows, int64_t in_features,
                                             hipengine_stream_t stream);

/* bf16 [rows, hidden] -> 144-byte DS4 blocks {half ds4[8]; int8 qs[128]},
 * [rows, hidden/128]: per 32 values scale = min(65504, amax/127),
 * q = clamp(rint(x/scale), -127, 127), ds4[2g] = half(scale), ds4[2g+1] = half(sum).
 * hidden % 128 == 0.
 * Replaces gguf_q4_k_q8_1_selected_prefill.hip:5582-5594 (kernel :627-690). */
int hipengine_gguf_q8_1_mmq_ds4_pack_bf16(const void* x, void* out, int64_t rows, int64_t hidden,
                                          hipengine_stream_t stream);

/* The same pack of rows gathered through the routing index, in one pass: output row r (of `rows` packed lanes)
 * is the pack of token sorted_lanes[r] / top_k of hidden_states [tokens, hidden]; a negative lane or a token
 * outside the input packs as a row of zeros.  Bytes equal hipengine_qwen35_moe_gather_packed_hidden_lowp followed
 * by the plain pack.  Replaces gguf_q4_k_q8_1_selected_prefill.hip:5596-5614 (kernel :705-772). */
int hipengine_gguf_q8_1_mmq_gather_ds4_pack_bf16(const uint16_t* hidden_states, const int64_t* sorted_lanes,
                                                 void* out, int64_t rows, int64_t hidden, int64_t tokens,
                                                 int64_t top_k, hipengine_stream_t stream);

/* bf16 [rows, hidden] -> 160-byte D4S4 blocks {float d4[4]; float s4[4]; int8 qs[128]}:
 * d = amax/127 (float32), q = clamp(roundf(x/d), -128, 127).  hidden % 128 == 0.
 * Replaces gguf_k_mmq_prefill.hip:2515-2540 (kernel :264-307). */
int hipengine_gguf_q8_1_d4s4_f32_quantize_bf16(const void* x, void* out, int64_t rows, int64_t hidden,
                                               hipengine_stream_t stream);

/* ------------------------------------------------------------------------
 * Decode GEMV, batch 1..8 per launch (more rows are split into launches of 8)
 *   out[r, n] = sum_k W[n, k] * x[r, k],  W raw Q4_K / Q5_K / Q6_K / Q8_0 blocks
 * in_features % 256 == 0 for all weight types.  Q5_K follows the arithmetic of gguf_k_gemv.hip:115-137 on q8_1
 * activations (the Q4_K formula with the fifth bit taken from qh) and takes every kernel form but the Q4_K slab.
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
HIPENGINE_GFX950_DECLARE_FUSED_ALL(q5_k)
HIPENGINE_GFX950_DECLARE_FUSED_ALL(q6_k)
HIPENGINE_GFX950_DECLARE_FUSED_ALL(q8_0)

/* hipEngine's own dense names, which its wrappers bind and its dispatcher reaches through the registry
 * keys ("linear", quant, "gemv_<act>_<out>_out") and, for rows > 1, ("linear", quant, "prefill_<act>_<out>_out")
 * (loading/qwen35_gguf_consumer_surface.py:134-144,527-530).  Same argument list; here they run the fused
 * kernels above, so the arithmetic is q8_1 activations x integer weights (what hipEngine's dp4a kernels
 * compute), not the float-activation arithmetic of hipEngine's kernels of the same name.  Any rows >= 1:
 * batches of up to 8 rows per launch; from 32 rows of bf16 activations on, the MMQ GEMM instead, in chunks of at
 * most 512 rows packed into a buffer the library holds (two regions per device used in turn: calls that overlap
 * on one device may not number more than two; results then follow the MMQ's DS4 / D4S4 activation format).
 * Replace gguf_q4_k_gemv.hip:2483-2611 (Q4_K) and gguf_k_gemv.hip:5504-5545 (Q5_K, Q6_K, Q8_0). */
#define HIPENGINE_GFX950_DECLARE_DENSE(q, a, o)                                                          \
  int hipengine_gguf_##q##_gemv_##a##_##o##_out(                                                         \
      const void* x, const uint8_t* qweight, void* out, int64_t rows, int64_t in_features,               \
      int64_t out_features, int64_t threads, hipengine_stream_t stream);
/* Two matrices over one activation, out_a = W_a x and out_b = W_b x (k and v, gate and up): one launch for
 * rows <= 2 and in_features >= 4096, and for Q4_K with in_features <= 6144 at rows 3..8, else one per matrix.
 * Replaces gguf_k_gemv.hip:5546-5560. */
#define HIPENGINE_GFX950_DECLARE_DENSE_DUAL(q, a, o)                                                     \
  int hipengine_gguf_##q##_dual_gemv_##a##_##o##_out(                                                    \
      const void* x, const uint8_t* qweight_a, const uint8_t* qweight_b, void* out_a, void* out_b,       \
      int64_t rows, int64_t in_features, int64_t out_features, int64_t threads, hipengine_stream_t stream);
/* The "rowtile" names of the same (hipEngine's kernels for 2 to 8 rows that reuse a weight row across the batch;
 * every batch here does): gguf_q4_k_gemv.hip:2496-2533, gguf_k_gemv.hip:5600-5617. */
#define HIPENGINE_GFX950_DECLARE_ROWTILE(q, a, o)                                                        \
  int hipengine_gguf_##q##_gemv_rowtile_##a##_##o##_out(                                                 \
      const void* x, const uint8_t* qweight, void* out, int64_t rows, int64_t in_features,               \
      int64_t out_features, int64_t threads, hipengine_stream_t stream);
#define HIPENGINE_GFX950_DECLARE_DENSE_ALL(q) \
  HIPENGINE_GFX950_DECLARE_ROWTILE(q, f32, f32) \
  HIPENGINE_GFX950_DECLARE_ROWTILE(q, bf16, f32) \
  HIPENGINE_GFX950_DECLARE_ROWTILE(q, bf16, bf16) \
  HIPENGINE_GFX950_DECLARE_DENSE(q, f32, f32) \
  HIPENGINE_GFX950_DECLARE_DENSE(q, f32, fp16) \
  HIPENGINE_GFX950_DECLARE_DENSE(q, fp16, f32) \
  HIPENGINE_GFX950_DECLARE_DENSE(q, fp16, fp16) \
  HIPENGINE_GFX950_DECLARE_DENSE(q, bf16, f32) \
  HIPENGINE_GFX950_DECLARE_DENSE(q, bf16, fp16) \
  HIPENGINE_GFX950_DECLARE_DENSE(q, bf16, bf16) \
  HIPENGINE_GFX950_DECLARE_DENSE_DUAL(q, f32, f32) \
  HIPENGINE_GFX950_DECLARE_DENSE_DUAL(q, bf16, bf16)
HIPENGINE_GFX950_DECLARE_DENSE_ALL(q4_k)
HIPENGINE_GFX950_DECLARE_DENSE_ALL(q5_k)
HIPENGINE_GFX950_DECLARE_DENSE_ALL(q6_k)
HIPENGINE_GFX950_DECLARE_DENSE_ALL(q8_0)

/* hipEngine's per-shape tuning variants of the dense GEMV for Q5_K / Q6_K / Q8_0 (row batches, column tiles, wave
 * layouts, pipelining; gguf_k_gemv.hip:5665-5702, 5823-5960, 6161-6255): the same 8 arguments and product as the
 * dense names above and the same launch here, for any shape (hipEngine restricts some to the shapes they were tuned
 * for).  The pair names take two Q5_K matrices of different heights over one bf16 activation. */
#define HIPENGINE_GFX950_DECLARE_DENSE_VARIANT(name)                                                     \
  int name(const void* x, const uint8_t* qweight, void* out, int64_t rows, int64_t in_features,          \
           int64_t out_features, int64_t threads, hipengine_stream_t stream);
#define HIPENGINE_GFX950_DECLARE_DENSE_VARIANT_BF16(prefix)        \
  HIPENGINE_GFX950_DECLARE_DENSE_VARIANT(prefix##_bf16_bf16_out)   \
  HIPENGINE_GFX950_DECLARE_DENSE_VARIANT(prefix##_bf16_f32_out)
HIPENGINE_GFX950_DECLARE_DENSE_VARIANT_BF16(hipengine_gguf_q5_k_gemv_rowbatch8)
HIPENGINE_GFX950_DECLARE_DENSE_VARIANT_BF16(hipengine_gguf_q5_k_gemv_rowbatch32)
HIPENGINE_GFX950_DECLARE_DENSE_VARIANT_BF16(hipengine_gguf_q6_k_gemv_rowbatch8)
HIPENGINE_GFX950_DECLARE_DENSE_VARIANT_BF16(hipengine_gguf_q6_k_gemv_rowbatch32)
HIPENGINE_GFX950_DECLARE_DENSE_VARIANT_BF16(hipengine_gguf_q5_k_gemv_coltile2_rowbatch16)
HIPENGINE_GFX950_DECLARE_DENSE_VARIANT_BF16(hipengine_gguf_q5_k_gemv_coltile4_rowbatch8)
HIPENGINE_GFX950_DECLARE_DENSE_VARIANT_BF16(hipengine_gguf_q6_k_gemv_coltile2_rowbatch16)
HIPENGINE_GFX950_DECLARE_DENSE_VARIANT_BF16(hipengine_gguf_q6_k_gemv_coltile4_rowbatch8)
HIPENGINE_GFX950_DECLARE_DENSE_VARIANT_BF16(hipengine_gguf_q5_k_wave32x2_gemv_decode)
HIPENGINE_GFX950_DECLARE_DENSE_VARIANT_BF16(hipengine_gguf_q5_k_wave32x2_fixed_meta_gemv_decode)
HIPENGINE_GFX950_DECLARE_DENSE_VARIANT_BF16(hipengine_gguf_q5_k_wave32x2_swar_pair_fixed_meta_gemv_decode)
HIPENGINE_GFX950_DECLARE_DENSE_VARIANT(hipengine_gguf_q6_k_wave32x2_fixed_meta_gemv_decode_bf16_bf16_out)
HIPENGINE_GFX950_DECLARE_DENSE_VARIANT(hipengine_gguf_q6_k_gemv_dpp_wave_reduction_coltile4_rowbatch8_bf16_bf16_out)
HIPENGINE_GFX950_DECLARE_DENSE_VARIANT(hipengine_gguf_q6_k_gemv_dpp_wave_reduction_coltile2_rowbatch16_bf16_f32_out)
HIPENGINE_GFX950_DECLARE_DENSE_VARIANT(hipengine_gguf_q6_k_gemv_dpp_wave_reduction_full_group_compute_coltile4_rowbatch8_bf16_bf16_out)
HIPENGINE_GFX950_DECLARE_DENSE_VARIANT(hipengine_gguf_q6_k_gemv_dpp_wave_reduction_full_group_compute_coltile2_rowbatch16_bf16_f32_out)
HIPENGINE_GFX950_DECLARE_DENSE_VARIANT(hipengine_gguf_q8_0_gemv_coltile4_rowbatch8_pipelined_f32_f32_out)
HIPENGINE_GFX950_DECLARE_DENSE_VARIANT(hipengine_gguf_q8_0_gemv_coltile8_rowbatch4_pipelined_f32_f32_out)
HIPENGINE_GFX950_DECLARE_DENSE_VARIANT(hipengine_gguf_q8_0_gemv_coltile8_rowbatch4_wave_scale_f32_f32_out)
HIPENGINE_GFX950_DECLARE_DENSE_VARIANT(hipengine_gguf_q8_0_gemv_coltile8_rowbatch4_wave_scale_pipelined_f32_f32_out)
HIPENGINE_GFX950_DECLARE_DENSE_VARIANT(hipengine_gguf_q8_0_gemv_coltile8_rowbatch4_wave_scale_pipelined_dpp_f32_f32_out)
HIPENGINE_GFX950_DECLARE_DENSE_VARIANT(hipengine_gguf_q8_0_gemv_coltile8_rowbatch4_wave_scale_pipelined_dpp_checked_full_rows_f32_f32_out)
#define HIPENGINE_GFX950_DECLARE_Q5_K_PAIR(name)                                                          \
  int name(const void* x, const uint8_t* qweight_a, const uint8_t* qweight_b, void* out_a, void* out_b, int64_t rows, \
           int64_t in_features, int64_t out_features_a, int64_t out_features_b, int64_t threads,           \
           hipengine_stream_t stream);
HIPENGINE_GFX950_DECLARE_Q5_K_PAIR(hipengine_gguf_q5_k_pair_wave32x2_gemv_decode_bf16_f32_out)
HIPENGINE_GFX950_DECLARE_Q5_K_PAIR(hipengine_gguf_q5_k_pair_wave32x2_fixed_meta_gemv_decode_bf16_bf16_out)
HIPENGINE_GFX950_DECLARE_Q5_K_PAIR(hipengine_gguf_q5_k_pair_wave32x2_fixed_meta_gemv_decode_bf16_f32_out)
HIPENGINE_GFX950_DECLARE_Q5_K_PAIR(hipengine_gguf_q5_k_pair_wave32x2_swar_pair_fixed_meta_gemv_decode_bf16_bf16_out)
HIPENGINE_GFX950_DECLARE_Q5_K_PAIR(hipengine_gguf_q5_k_pair_wave32x2_swar_pair_fixed_meta_gemv_decode_bf16_f32_out)

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
/* The "ctl" names of the same Q4_K kernel (gguf_q4_k_q8_1_dp4a_vdr_gemv.hip:348-364: a second code shape of the
 * same arithmetic in hipEngine; one kernel here). */
int hipengine_gguf_q4_k_q8_1_dp4a_ctl_bf16_f32_out(const void* xq, const uint8_t* qweight, void* out, int64_t rows,
                                                   int64_t in_features, int64_t out_features,
                                                   hipengine_stream_t stream);
int hipengine_gguf_q4_k_q8_1_dp4a_ctl_bf16_bf16_out(const void* xq, const uint8_t* qweight, void* out, int64_t rows,
                                                    int64_t in_features, int64_t out_features,
                                                    hipengine_stream_t stream);

/* Q8_0 weights over pre-quantized q8_1 activations (gguf_q8_0_dp4a_gemv.hip:345-387).  As in hipEngine these
 * carry a `threads` argument before the stream, which is ignored.  The "rowtile4" names (lines 389-437) are
 * hipEngine's variant that reuses a weight row across four activation rows; here every batch already does,
 * so they run the same kernels.  in_features must be a multiple of 256 (hipEngine: of 32). */
int hipengine_gguf_q8_0_dp4a_gemv_f32_f32_out(const void* xq, const uint8_t* qweight, void* out, int64_t rows,
                                              int64_t in_features, int64_t out_features, int64_t threads,
                                              hipengine_stream_t stream);
int hipengine_gguf_q8_0_dp4a_gemv_bf16_bf16_out(const void* xq, const uint8_t* qweight, void* out, int64_t rows,
                                                int64_t in_features, int64_t out_features, int64_t threads,
                                                hipengine_stream_t stream);
int hipengine_gguf_q8_0_dp4a_rowtile4_gemv_f32_f32_out(const void* xq, const uint8_t* qweight, void* out, int64_t rows,
                                                       int64_t in_features, int64_t out_features, int64_t threads,
                                                       hipengine_stream_t stream);
int hipengine_gguf_q8_0_dp4a_rowtile4_gemv_bf16_bf16_out(const void* xq, const uint8_t* qweight, void* out,
                                                         int64_t rows, int64_t in_features, int64_t out_features,
                                                         int64_t threads, hipengine_stream_t stream);

/* Two or three Q8_0 matrices over the same q8_1 activations, each with its own contiguous output
 * [rows, out_features_i] (gguf_q8_0_dp4a_gemv.hip:439-600: the q/k/v or gate/up projections of a block in one
 * launch).  rows <= 2 take one launch of the streaming kernel shared among the matrices by their sizes; larger
 * batches run one launch per matrix.  Every output is bit-equal to the single-matrix call's. */
int hipengine_gguf_q8_0_dp4a_dual_split_rowtile4_gemv_f32_f32_out(const void* xq, const uint8_t* qweight_a,
                                                                  const uint8_t* qweight_b, void* out_a, void* out_b,
                                                                  int64_t rows, int64_t in_features,
                                                                  int64_t out_features_a, int64_t out_features_b,
                                                                  int64_t threads, hipengine_stream_t stream);
int hipengine_gguf_q8_0_dp4a_dual_split_rowtile4_gemv_bf16_bf16_out(const void* xq, const uint8_t* qweight_a,
                                                                    const uint8_t* qweight_b, void* out_a, void* out_b,
                                                                    int64_t rows, int64_t in_features,
                                                                    int64_t out_features_a, int64_t out_features_b,
                                                                    int64_t threads, hipengine_stream_t stream);
int hipengine_gguf_q8_0_dp4a_triple_split_rowtile4_gemv_f32_f32_out(
    const void* xq, const uint8_t* qweight_a, const uint8_t* qweight_b, const uint8_t* qweight_c, void* out_a,
    void* out_b, void* out_c, int64_t rows, int64_t in_features, int64_t out_features_a, int64_t out_features_b,
    int64_t out_features_c, int64_t threads, hipengine_stream_t stream);
int hipengine_gguf_q8_0_dp4a_triple_split_rowtile4_gemv_bf16_bf16_out(
    const void* xq, const uint8_t* qweight_a, const uint8_t* qweight_b, const uint8_t* qweight_c, void* out_a,
    void* out_b, void* out_c, int64_t rows, int64_t in_features, int64_t out_features_a, int64_t out_features_b,
    int64_t out_features_c, int64_t threads, hipengine_stream_t stream);

/* Up to four matrices over one activation, out_i = W_i x: the q, k and v projections of an attention block,
 * whatever their types (each of Q4_K, Q5_K, Q6_K, Q8_0) and row counts.  qweights, outs and out_features are
 * host arrays of `count` entries, read before the call returns; x [rows, in_features] of x_kind, every out_i
 * [rows, out_features[i]] of out_kind.  rows <= 2 and in_features >= 4096: one launch, the workgroups divided
 * between the matrices in proportion to their bytes, each matrix computed in the stream form (the float32 sums
 * of its own call wherever that takes the stream form too).  rows 3..8: the Q4_K matrices with in_features <= 6144
 * share one launch of the slab form (the 256 workgroups divided in proportion to their rows; the bits of their
 * own calls), the others take a launch each.  Otherwise one launch per matrix.  hipEngine has the form for
 * two and three Q8_0 matrices (gguf_q8_0_dp4a_gemv.hip:100-340).  New here. */
int hipengine_gfx950_gguf_multi_gemv(int32_t count, const int32_t* ggml_types, const void* x, int32_t x_kind,
                                     const uint8_t* const* qweights, void* const* outs, int32_t out_kind,
                                     int64_t rows, int64_t in_features, const int64_t* out_features,
                                     hipengine_stream_t stream);

/* Gate/up pair of a dense FFN with SiLU*up fused: out[r, n] = silu(gate_n . x_r) * (up_n . x_r), one pass
 * over both matrices, q8_1 quantization of x fused.  round_mid != 0 rounds gate and up to the output type
 * before the SiLU, which reproduces the unfused sequence GEMV, GEMV, silu_mul on stored values
 * (arithmetic of gguf_q4_k_gemv.hip:652-657; hipEngine fuses this for its pack8 layout only,
 * hipengine_gguf_q4_k_pack8_dual_silu_gemv_bf16_bf16_out, and launch_gguf_linear_pair_silu
 * (runtime/qwen35_gguf_layer_ffn.py:519-538) falls back to the unfused sequence when no fused kernel
 * applies; so must a caller here when this returns 1).  rows <= 2: Q4_K, in_features >= 4096 and
 * out_features large enough for the stream form (a 27B FFN is), one launch.  rows 3..8: any of the four
 * types on the int8 MFMA forms, out = silu(round(gate)) * round(up) with both rounded to the output type
 * (the round_mid arithmetic: a 16-bit out_kind needs round_mid != 0) - one launch for Q4_K with
 * in_features <= 6144 and out_features <= 72 * 256 (a workgroup walks its rows of the gate matrix, then the
 * same rows of the up matrix), else a gate launch that stores to `out` and an up launch whose epilogue reads
 * it back; both give the same bits.  New here. */
int hipengine_gfx950_gguf_pair_silu_gemv(int32_t ggml_type, const void* x, int32_t x_kind, const uint8_t* qweight_gate,
                                         const uint8_t* qweight_up, void* out, int32_t out_kind, int64_t rows,
                                         int64_t in_features, int64_t out_features, int32_t round_mid,
                                         hipengine_stream_t stream);

/* Projection with the residual add fused: out = round_to_out_type(W x) + residual, residual [rows, N] of the
 * output type (may be the same buffer as out) - the epilogue of
 * hipengine_gguf_q4_k_pack8_gemv_bf16_residual_bf16_out (gguf_q4_k_gemv.hip:1669-1678, :3080-3110) on the raw
 * layout.  Q4_K in the slab form's range (any rows <= 8), Q4_K / Q6_K in the stream form's range (rows <= 2);
 * returns 1 otherwise, and the caller runs the GEMV and the add separately.  New here. */
int hipengine_gfx950_gguf_gemv_residual(int32_t ggml_type, const void* x, int32_t x_kind, const uint8_t* qweight,
                                        const void* residual, void* out, int32_t out_kind, int64_t rows,
                                        int64_t in_features, int64_t out_features, hipengine_stream_t stream);

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

/* Raw Q5_K weights x D4S4 activations ([rows, in_features/128] 160-byte blocks, float32 scale and raw sum per
 * 32 values): sum_j (d*sc_j)*xd_j*dot_j - (dmin*mn_j)*s4_j per 32-wide sub-block, dot of the 5-bit values.
 * Replaces gguf_k_mmq_prefill.hip:2557-2589 with NAME = gguf_q5_k (kernel :517-685, qtype 5); the pipe and mb4
 * names of the same export block are scheduling variants of this kernel there and are not exported here. */
int hipengine_gguf_q5_k_mmq32_q8_1_d4s4_f32_bf16_f32_out(const void* xq, const uint8_t* qweight, void* out,
                                                         int64_t rows, int64_t in_features, int64_t out_features,
                                                         hipengine_stream_t stream);
int hipengine_gguf_q5_k_mmq32_q8_1_d4s4_f32_bf16_bf16_out(const void* xq, const uint8_t* qweight, void* out,
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

/* hipEngine's scheduling variants of the two GEMMs above (gguf_k_mmq_prefill.hip:2565-2578 "pipe" and "mb4",
 * :2315-2366 "direct_dp4a"): the same arguments and results from the one kernel form here (Q5_K: out_features % 32
 * == 0, which hipEngine's direct_dp4a form does not ask for). */
int hipengine_gguf_q5_k_mmq32_pipe_q8_1_d4s4_f32_bf16_bf16_out(const void* xq, const uint8_t* qweight, void* out,
                                                               int64_t rows, int64_t in_features,
                                                               int64_t out_features, hipengine_stream_t stream);
int hipengine_gguf_q5_k_mmq32_mb4_q8_1_d4s4_f32_bf16_bf16_out(const void* xq, const uint8_t* qweight, void* out,
                                                              int64_t rows, int64_t in_features, int64_t out_features,
                                                              hipengine_stream_t stream);
int hipengine_gguf_q5_k_mmq32_direct_dp4a_q8_1_d4s4_f32_bf16_bf16_out(const void* xq, const uint8_t* qweight, void* out,
                                                                      int64_t rows, int64_t in_features,
                                                                      int64_t out_features, hipengine_stream_t stream);
int hipengine_gguf_q5_k_mmq32_direct_dp4a_q8_1_d4s4_f32_bf16_f32_out(const void* xq, const uint8_t* qweight, void* out,
                                                                     int64_t rows, int64_t in_features,
                                                                     int64_t out_features, hipengine_stream_t stream);
int hipengine_gguf_q6_k_mmq32_pipe_q8_1_d4s4_f32_bf16_bf16_out(const void* xq, const uint8_t* qweight, void* out,
                                                               int64_t rows, int64_t in_features,
                                                               int64_t out_features, hipengine_stream_t stream);
int hipengine_gguf_q6_k_mmq32_mb4_q8_1_d4s4_f32_bf16_bf16_out(const void* xq, const uint8_t* qweight, void* out,
                                                              int64_t rows, int64_t in_features, int64_t out_features,
                                                              hipengine_stream_t stream);

/* Raw Q8_0 weights ([out_features, in_features/32 * 34]) x D4S4 activations: sum over the 32-value blocks of
 * xd_b * d_b * dot_b, the q8_1 x Q8_0 formula (gguf_q8_0_dp4a_gemv.hip:100-137) with the float32 activation scales
 * of the D4S4 block, on the int8 MFMA.  in_features a multiple of 128; any out_features >= 1.  hipEngine has no MMQ
 * for Q8_0 (its Q8_0 prefill names run the GEMV over row chunks); named after the k-quant MMQ entries.  New here. */
int hipengine_gguf_q8_0_mmq32_q8_1_d4s4_f32_bf16_f32_out(const void* xq, const uint8_t* qweight, void* out,
                                                         int64_t rows, int64_t in_features, int64_t out_features,
                                                         hipengine_stream_t stream);
int hipengine_gguf_q8_0_mmq32_q8_1_d4s4_f32_bf16_bf16_out(const void* xq, const uint8_t* qweight, void* out,
                                                          int64_t rows, int64_t in_features, int64_t out_features,
                                                          hipengine_stream_t stream);

/* Prefill from bf16 activations in one call: x [rows, in_features] bf16 is packed into `workspace`
 * (DS4 blocks for Q4_K, D4S4 for Q5_K, Q6_K and Q8_0; caller-owned, 16-byte aligned, at least the byte count
 * hipengine_gfx950_gguf_prefill_workspace_bytes reports = rows * in_features/128 * 144 or 160) and the MMQ
 * above runs on it: two launches.  ggml_type 12 (Q4_K), 13 (Q5_K; both out_features % 32 == 0), 14 (Q6_K) or 8
 * (Q8_0, in_features % 128 == 0); out_kind 0
 * float32, 1 bf16, 2 fp16.  The dense names above reach the same GEMM from 32 rows on through the library's own
 * pack buffer (hipEngine's prefill signature has no workspace argument); this entry is for a caller that wants
 * all rows packed at once into memory of its own - no limit on overlapping calls, one GEMM launch - and the
 * Python wrappers of the prefill keys take such a workspace as an optional keyword.  Same bits either way.
 * New here. */
int hipengine_gfx950_gguf_prefill_workspace_bytes(int32_t ggml_type, int64_t rows, int64_t in_features,
                                                  int64_t* bytes);
int hipengine_gfx950_gguf_prefill_bf16(int32_t ggml_type, const void* x, const uint8_t* qweight, void* out,
                                       int32_t out_kind, int64_t rows, int64_t in_features, int64_t out_features,
                                       void* workspace, int64_t workspace_bytes, hipengine_stream_t stream);

/* ------------------------------------------------------------------------
 * MoE: routing index, expert-indexed decode GEMV, expert-grouped prefill MMQ
 * Expert weights are [num_experts, out_features, row_bytes] raw blocks.
 * A lane is one (token, slot) pair: lane = token * top_k + slot.
 * num_experts <= 2048.
 * ------------------------------------------------------------------------ */

/* Token embedding lookup over raw GGUF rows: out[r, 0..hidden_size) = bf16(dequantize(row token_ids[r] of
 * qweight)), qweight [vocab_size, hidden_size / block * block_bytes].  A row whose token id is outside
 * [0, vocab_size) is left untouched.  hidden_size % 256 == 0 (Q8_0: % 32); `threads` is accepted and ignored.
 * Replace hipengine_gguf_{q4_k,q5_k,q6_k,q8_0}_embedding_bf16_out
 * (kernels/hip_gfx1100/quant/gguf_q6_k_embedding.hip:240-350). */
int hipengine_gguf_q4_k_embedding_bf16_out(const int64_t* token_ids, const uint8_t* qweight, uint16_t* out,
                                           int64_t rows, int64_t hidden_size, int64_t vocab_size, int64_t threads,
                                           hipengine_stream_t stream);
int hipengine_gguf_q5_k_embedding_bf16_out(const int64_t* token_ids, const uint8_t* qweight, uint16_t* out,
                                           int64_t rows, int64_t hidden_size, int64_t vocab_size, int64_t threads,
                                           hipengine_stream_t stream);
int hipengine_gguf_q6_k_embedding_bf16_out(const int64_t* token_ids, const uint8_t* qweight, uint16_t* out,
                                           int64_t rows, int64_t hidden_size, int64_t vocab_size, int64_t threads,
                                           hipengine_stream_t stream);
int hipengine_gguf_q8_0_embedding_bf16_out(const int64_t* token_ids, const uint8_t* qweight, uint16_t* out,
                                           int64_t rows, int64_t hidden_size, int64_t vocab_size, int64_t threads,
                                           hipengine_stream_t stream);

/* Row-wise arg-max of float32 logits [rows, vocab_size] (greedy decode after the lm_head GEMV): the highest
 * value's index (lowest index among equal values) as int32 into out_indices[rows], the value into out_values
 * when that is not null.  block_values / block_indices are caller-owned scratch of
 * rows * ceil(vocab_size / (threads * 4)) entries; threads in {128, 256, 512}.
 * Replaces hipengine_argmax_f32_rows_i32 (kernels/hip_gfx1100/linear/lm_head.hip:746-793). */
int hipengine_argmax_f32_rows_i32(const float* logits, float* block_values, int32_t* block_indices,
                                  int32_t* out_indices, float* out_values, int64_t rows, int64_t vocab_size,
                                  int64_t threads, hipengine_stream_t stream);

/* The same arg-max for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc): the stage scratch is a fixed array inside the library
 * instead of two caller buffers.  It has no counterpart in hipEngine.  Same results as
 * hipengine_argmax_f32_rows_i32 with the same `threads`.  Limit: rows * ceil(vocab_size / (threads * 4))
 * <= HIPENGINE_GFX950_ARGMAX_NOALLOC_MAX_ENTRIES, otherwise hipErrorInvalidValue (1) and nothing is
 * launched.  The array (512 KiB per device, held until the process ends) is shared by every call on a
 * device: calls that overlap on one device - different streams, or two graphs replayed concurrently -
 * race on it; calls in stream order do not.  No call allocates, frees or synchronizes; the first call on
 * a device looks up the array's address unless hipengine_gfx950_init() has done so. */
#define HIPENGINE_GFX950_ARGMAX_NOALLOC_MAX_ENTRIES 65536
int hipengine_gfx950_argmax_f32_rows_i32_noalloc(const float* logits, int32_t* out_indices, float* out_values,
                                                 int64_t rows, int64_t vocab_size, int64_t threads,
                                                 hipengine_stream_t stream);

/* Router logits, the product in front of the selection: logits[t, e] = hidden[t, :] . weight[e, :] accumulated in
 * float32 (moe/router.hip:36-80, entries :960-1037,1140-1160,1250-1275).  hidden [tokens, hidden_size] in bf16, fp16 or
 * float32; weight [num_rows, hidden_size] in the same 16-bit type or in float32 (`_f32w`); logits float32
 * [tokens, num_rows].  Rows of 8 values or more must be 16-byte aligned (hidden_size * element size a multiple of
 * 16).  `threads` (64, 128, 256 or 512) is accepted and ignored.  Sums are taken in another order than hipEngine's
 * shared-memory tree: equal to float32 rounding. */
int hipengine_qwen35_router_logits_bf16(const void* hidden, const void* weight, float* logits, int64_t tokens,
                                        int64_t hidden_size, int64_t num_rows, int64_t threads,
                                        hipengine_stream_t stream);
int hipengine_qwen35_router_logits_fp16(const void* hidden, const void* weight, float* logits, int64_t tokens,
                                        int64_t hidden_size, int64_t num_rows, int64_t threads,
                                        hipengine_stream_t stream);
int hipengine_qwen35_router_logits_bf16_f32w(const void* hidden, const void* weight, float* logits, int64_t tokens,
                                             int64_t hidden_size, int64_t num_rows, int64_t threads,
                                             hipengine_stream_t stream);
int hipengine_qwen35_router_logits_fp16_f32w(const void* hidden, const void* weight, float* logits, int64_t tokens,
                                             int64_t hidden_size, int64_t num_rows, int64_t threads,
                                             hipengine_stream_t stream);
int hipengine_qwen35_router_logits_f32_f32w(const void* hidden, const void* weight, float* logits, int64_t tokens,
                                            int64_t hidden_size, int64_t num_rows, int64_t threads,
                                            hipengine_stream_t stream);

/* Router: for each of `tokens` rows of float32 logits (row pitch logits_stride), the top_k
 * experts by logit, highest first (equal logits: lowest index), as int64 into
 * selected[tokens*top_k], and the softmax over those top_k logits into
 * routing[tokens*top_k].  top_k <= 16, num_experts <= 1024; `threads` in {64,128,256,512}
 * is accepted and ignored.
 * Deviation on exact ties only: hipEngine's kernel strides the experts over `threads` threads and keeps
 * the first maximum a thread meets, then the first over threads; with num_experts > threads two equal
 * logits can there resolve to the higher index (expert 259 on thread 3 before expert 5 on thread 5 at
 * 256 threads).  Here equal logits always go to the lowest index, whatever `threads` is; with
 * num_experts <= threads the two orders are the same.
 * Replaces hipengine_qwen35_router_select (kernels/hip_gfx1100/moe/router.hip:1284-1311,
 * device function :628-715). */
int hipengine_qwen35_router_select(const float* logits, int64_t* selected, float* routing, int64_t tokens,
                                   int64_t logits_stride, int64_t num_experts, int64_t top_k, int64_t threads,
                                   hipengine_stream_t stream);

/* selected_experts[total_lanes] -> expert-major order.  expert_start[num_experts+1]
 * (exclusive prefix of the per-expert lane counts), active_experts (ascending ids
 * of experts with at least one lane; may be NULL) and active_count[1] (may be NULL),
 * sorted_lanes[total_lanes] (ascending lane within an expert), sorted_experts (may
 * be NULL), sorted_weights (may be NULL).  Expert ids outside [0, num_experts) are
 * dropped.  Replaces moe/group_scatter.hip:760-797 (kernel :85-141). */
int hipengine_qwen35_moe_group_compact_active(const int64_t* selected_experts, const float* routing_weights,
                                              int64_t* expert_start, int64_t* active_experts, int64_t* active_count,
                                              int64_t* sorted_lanes, int64_t* sorted_experts, float* sorted_weights,
                                              int64_t total_lanes, int64_t num_experts, hipengine_stream_t stream);

/* The same with compact_to_source[i] = sorted_lanes[i] / top_k instead of
 * sorted_experts.  Replaces moe/group_scatter.hip:799-836. */
int hipengine_qwen35_moe_group_compact_active_source_rows(const int64_t* selected_experts,
                                                          const float* routing_weights, int64_t* expert_start,
                                                          int64_t* active_experts, int64_t* active_count,
                                                          int64_t* sorted_lanes, int64_t* compact_to_source,
                                                          float* sorted_weights, int64_t total_lanes,
                                                          int64_t num_experts, int64_t top_k,
                                                          hipengine_stream_t stream);

/* The step-by-step form of the same index, as hipEngine's runner drives it
 * (runtime/qwen35_gguf_runner.py:34107-34143): count, prefix, scatter + gather.
 *   group_count   counts[e] (int32, zeroed by the caller) += lanes whose expert is e.
 *                 Replaces moe/group_scatter.hip:683-705 (kernel :9-22).
 *   group_prefix  padded_counts[e] = counts[e] rounded up to pad_multiple; expert_start[0..E] = exclusive
 *                 prefix of the padded counts; total_padded[0] = their sum.  num_experts <= 2048.
 *                 Replaces moe/group_scatter.hip:707-733 (kernel :24-60).
 *   group_scatter_gather_lowp  for every lane with a valid expert e: a slot i in
 *                 [expert_start[e] + scatter_offsets[e], ...) gets sorted_lanes[i] = lane, sorted_experts[i] = e,
 *                 sorted_weights[i] = routing_weights[lane] and packed_hidden[i, :] = hidden_states[lane / top_k, :]
 *                 (16-bit elements); scatter_offsets[e] (int32, zeroed by the caller) ends as the number of
 *                 lanes placed.  hipEngine takes slots with atomics, in arrival order; here an expert's lanes
 *                 are placed in ascending lane order, which is one of the orders it can produce and makes the
 *                 result deterministic.  Replaces moe/group_scatter.hip:1121-1159 (kernel :419-460).
 *   gather_packed_hidden_lowp  packed_hidden[r, :] = hidden_states[sorted_lanes[r] / top_k, :] for the
 *                 total_elements / hidden_size rows, zeros where the lane is negative or its token is not in
 *                 [0, tokens).  Replaces moe/group_scatter.hip:1161-1206 (kernel :462-485). */
int hipengine_qwen35_moe_group_count(const int64_t* selected_experts, int32_t* counts, int64_t total_lanes,
                                     int64_t num_experts, hipengine_stream_t stream);
int hipengine_qwen35_moe_group_prefix(const int32_t* counts, int32_t* padded_counts, int64_t* expert_start,
                                      int64_t* total_padded, int64_t num_experts, int64_t pad_multiple,
                                      hipengine_stream_t stream);
int hipengine_qwen35_moe_group_scatter_gather_lowp(const uint16_t* hidden_states, const int64_t* selected_experts,
                                                   const float* routing_weights, const int64_t* expert_start,
                                                   int32_t* scatter_offsets, int64_t* sorted_lanes,
                                                   int64_t* sorted_experts, float* sorted_weights,
                                                   uint16_t* packed_hidden, int64_t total_lanes, int64_t num_experts,
                                                   int64_t top_k, int64_t hidden_size, hipengine_stream_t stream);
int hipengine_qwen35_moe_gather_packed_hidden_lowp(const uint16_t* hidden_states, const int64_t* sorted_lanes,
                                                   uint16_t* packed_hidden, int64_t total_elements, int64_t tokens,
                                                   int64_t top_k, int64_t hidden_size, hipengine_stream_t stream);

/* expert_start_compact[num_experts+1] -> mmq_expert_start[num_experts+1] (row
 * starts with every expert's count rounded up to 32), tile_expert[tile] (expert
 * of each 32-row tile; the first tile_capacity entries are preset to -1 when
 * tile_capacity > 0 and tiles beyond it are not written), mmq_total_out[1].
 * Replaces moe/group_scatter.hip:1023-1052 (kernel :328-389). */
int hipengine_qwen35_moe_mmq32_tile_map(const int64_t* expert_start_compact, int64_t* mmq_expert_start,
                                        int64_t* tile_expert, int64_t* mmq_total_out, int64_t num_experts,
                                        int64_t tile_capacity, hipengine_stream_t stream);

/* The same map for hipEngine's other tile heights: 16 rows (moe/group_scatter.hip:994-1021) and 64 (:1054-1083). */
int hipengine_qwen35_moe_wmma_tile_map(const int64_t* expert_start_compact, int64_t* wmma_expert_start,
                                       int64_t* tile_expert, int64_t* wmma_total_out, int64_t num_experts,
                                       int64_t tile_capacity, hipengine_stream_t stream);
int hipengine_qwen35_moe_mmq64_tile_map(const int64_t* expert_start_compact, int64_t* mmq_expert_start,
                                        int64_t* tile_expert, int64_t* mmq_total_out, int64_t num_experts,
                                        int64_t tile_capacity, hipengine_stream_t stream);

/* hipEngine's "parallel" compaction names (moe/group_scatter.hip:909-992): the arrays of the stable compaction above,
 * which they equal there too (one workgroup per expert, ascending lanes); the i32 form takes int32 expert ids. */
int hipengine_qwen35_moe_group_compact_active_parallel(const int64_t* selected_experts, const float* routing_weights,
                                                       int64_t* expert_start, int64_t* active_experts,
                                                       int64_t* active_count, int64_t* sorted_lanes,
                                                       int64_t* sorted_experts, float* sorted_weights,
                                                       int64_t total_lanes, int64_t num_experts,
                                                       hipengine_stream_t stream);
int hipengine_qwen35_moe_group_compact_active_source_rows_parallel(
    const int64_t* selected_experts, const float* routing_weights, int64_t* expert_start, int64_t* active_experts,
    int64_t* active_count, int64_t* sorted_lanes, int64_t* compact_to_source, float* sorted_weights,
    int64_t total_lanes, int64_t num_experts, int64_t top_k, hipengine_stream_t stream);
int hipengine_qwen35_moe_group_compact_active_i32_parallel(const int32_t* selected_experts, const float* routing_weights,
                                                           int64_t* expert_start, int64_t* active_experts,
                                                           int64_t* active_count, int64_t* sorted_lanes,
                                                           int64_t* sorted_experts, float* sorted_weights,
                                                           int64_t total_lanes, int64_t num_experts,
                                                           hipengine_stream_t stream);

/* int32 counts [num_experts] -> expert_start [num_experts + 1] (exclusive prefix), the ascending list of the experts
 * with a positive count and their number (moe/group_scatter.hip:735-758). */
int hipengine_qwen35_moe_group_prefix_active(const int32_t* counts, int64_t* expert_start, int64_t* active_experts,
                                             int64_t* active_count, int64_t num_experts, hipengine_stream_t stream);

/* Scatter of the lanes into per-expert order from given starts; scatter_offsets [num_experts] is zeroed by the caller
 * and ends as the per-expert counts (moe/group_scatter.hip:1085-1118).  hipEngine takes an expert's slots with atomics
 * in arrival order; here its lanes land in ascending order (one of those orders, and a deterministic one). */
int hipengine_qwen35_moe_group_scatter(const int64_t* selected_experts, const float* routing_weights,
                                       const int64_t* expert_start, int32_t* scatter_offsets, int64_t* sorted_lanes,
                                       int64_t* sorted_experts, float* sorted_weights, int64_t total_lanes,
                                       int64_t num_experts, bool include_routing_weights, hipengine_stream_t stream);

/* lane_to_compact[total_lanes]: position of each lane in sorted_lanes, -1 for a
 * dropped lane.  New here (hipEngine scatters with atomics instead,
 * moe/group_scatter.hip:391-417; this inverse keeps the weighted sum ordered). */
int hipengine_gfx950_moe_lane_to_compact(const int64_t* sorted_lanes, int64_t* lane_to_compact, int64_t compact_rows,
                                         int64_t total_lanes, hipengine_stream_t stream);

/* hipengine_qwen35_moe_group_compact_active_source_rows and hipengine_gfx950_moe_lane_to_compact in the two
 * launches of the former: the placement writes lane_to_compact[lane] as it files the lane, the counting pass
 * writes -1 for the lanes of no expert.  Same arrays, bit for bit.  New here. */
int hipengine_gfx950_moe_group_compact_index(const int64_t* selected_experts, const float* routing_weights,
                                             int64_t* expert_start, int64_t* active_experts, int64_t* active_count,
                                             int64_t* sorted_lanes, int64_t* compact_to_source, float* sorted_weights,
                                             int64_t* lane_to_compact, int64_t total_lanes, int64_t num_experts,
                                             int64_t top_k, hipengine_stream_t stream);

/* gate_up[rows, 2*inter] (gate columns first) -> out[rows, inter] = gate*sigmoid(gate)*up.
 * Kinds: 0 float32, 1 bf16, 2 fp16.  The step between the gate/up and the down
 * projection (fused/paro_silu silu_mul_separate_out_bf16 in hipEngine). */
int hipengine_gfx950_moe_silu_mul(const void* gate_up, void* out, int64_t rows, int64_t inter, int in_kind,
                                  int out_kind, hipengine_stream_t stream);

/* gate_up[rows, 2*inter] -> DS4 blocks [rows, inter/128] of bf16(gate*sigmoid(gate)*up):
 * byte for byte what hipengine_gfx950_moe_silu_mul (bf16 out) followed by
 * hipengine_gguf_q8_1_mmq_ds4_pack_bf16 writes, in one launch.  inter % 128 == 0.
 * (hipEngine fuses the same pair in its ds4_f32 pack_dual_silu kernels,
 * gguf_q4_k_q8_1_selected_prefill.py:77-84.) */
int hipengine_gfx950_moe_silu_mul_ds4_pack(const void* gate_up, int in_kind, void* out, int64_t rows, int64_t inter,
                                           hipengine_stream_t stream);

/* The same into 160-byte D4S4 blocks (byte for byte hipengine_gfx950_moe_silu_mul with bf16 out followed by
 * hipengine_gguf_q8_1_d4s4_f32_quantize_bf16): the activations of a Q5_K / Q6_K down projection.  New here. */
int hipengine_gfx950_moe_silu_mul_d4s4_pack(const void* gate_up, int in_kind, void* out, int64_t rows, int64_t inter,
                                            hipengine_stream_t stream);

/* out[t, h] = sum over slots s = 0..top_k-1, in that order, of
 * routing_weights[t*top_k+s] * down[lane_to_compact[t*top_k+s], h]; lanes mapped
 * to -1 are skipped.  tokens <= 65535.  New here (see lane_to_compact). */
int hipengine_gfx950_moe_weighted_gather_sum(const void* down, const int64_t* lane_to_compact,
                                             const float* routing_weights, void* out, int64_t tokens, int64_t top_k,
                                             int64_t hidden, int64_t compact_rows, int in_kind, int out_kind,
                                             hipengine_stream_t stream);

/* The MoE tail fused with the next layer's RMSNorm, bf16 rows and a float32 norm weight
 * (kernels/hip_gfx1100/fused/paro_combine.hip:1505-1579; arithmetic of kernels/cpu_reference/ops.py:33-102):
 *   residual_out = bf16((residual + selected) + sigmoid(gate_logits[token * gate_stride]) * shared)
 *   norm_out     = bf16(residual_out / sqrt(mean(residual_out^2) + eps) * norm_weight)
 * `selected` [tokens, features] is the routed sum, already rounded to bf16.  residual_out may be residual itself.
 * One workgroup per token; 16-byte accesses when features % 8 == 0, features <= 8192 and the pointers are 16-byte
 * aligned, any other shape one value at a time.  Products and sums are rounded separately, as the CPU reference
 * does (hipEngine's HIP kernel lets the compiler contract them: results differ in the last bf16 bit now and then). */
int hipengine_shared_gate_combine_residual_rmsnorm_gguf_bf16_out(
    const uint16_t* selected, const uint16_t* shared, const float* gate_logits, const uint16_t* residual,
    const float* norm_weight, uint16_t* norm_out, uint16_t* residual_out, int64_t tokens, int64_t features,
    int64_t gate_stride, float eps, hipengine_stream_t stream);

/* The same with the routed sum formed here (kernels/hip_gfx1100/fused/paro_combine.hip:1542-1579): slot rows
 * selected_values [tokens * rows_per_token, features] (bf16) and routing_weights [tokens * rows_per_token],
 * acc = acc + value * weight in float32 in slot order, rounded to bf16 before it is added.  rows_per_token <= 4096. */
int hipengine_weighted_sum_shared_gate_combine_residual_rmsnorm_gguf_bf16_out(
    const uint16_t* selected_values, const float* routing_weights, const uint16_t* shared, const float* gate_logits,
    const uint16_t* residual, const float* norm_weight, uint16_t* norm_out, uint16_t* residual_out, int64_t tokens,
    int64_t rows_per_token, int64_t features, int64_t gate_stride, float eps, hipengine_stream_t stream);

/* The same over the compact rows of the grouped down projection: slot s of token t reads row
 * lane_to_compact[t * top_k + s] of down [compact_rows, features]; an entry outside [0, compact_rows) contributes
 * nothing.  Replaces hipengine_gfx950_moe_weighted_gather_sum followed by the tail.  New here. */
int hipengine_gfx950_moe_gather_tail_rmsnorm_bf16(
    const uint16_t* down, const int64_t* lane_to_compact, const float* routing_weights, const uint16_t* shared,
    const float* gate_logits, const uint16_t* residual, const float* norm_weight, uint16_t* norm_out,
    uint16_t* residual_out, int64_t tokens, int64_t top_k, int64_t features, int64_t compact_rows, int64_t gate_stride,
    float eps, hipengine_stream_t stream);

/* Decode: out[lane, :] = W[selected[lane]] . x[lane / (rows / x_rows), :] for
 * rows lanes (<= 65535) over x_rows activation rows; lanes with an expert id
 * outside [0, num_experts) are left unwritten.  Activations are quantized to
 * q8_1 in the kernel.  `threads` is accepted and ignored.
 * Replaces gguf_q4_k_gemv.hip selected GEMV export (kernel :322-359; Python
 * gguf_q4_k_gemv.py:667-715,1403). */
int hipengine_gguf_q4_k_selected_gemv_bf16_bf16_out(const uint16_t* x, const int64_t* selected,
                                                    const uint8_t* qweight, uint16_t* out, int64_t x_rows,
                                                    int64_t rows, int64_t num_experts, int64_t in_features,
                                                    int64_t out_features, int64_t threads,
                                                    hipengine_stream_t stream);

/* The same for Q5_K, Q6_K and Q8_0 experts (gguf_k_gemv.hip:5586-5592, macro instances :5619-5621), and their
 * down projection that takes the gate and up rows [x_rows, in_features] (bf16) as they are: the activation of
 * lane r is bf16(silu(gate) * up) of row r / (rows / x_rows), silu(g) = g / (1 + expf(-g)), formed while the
 * activations are staged and quantized to q8_1 (gguf_k_gemv.hip:5593-5599, kernel :1813-1866). */
#define HIPENGINE_GFX950_DECLARE_SELECTED_K(q)                                                                     \
  int hipengine_gguf_##q##_selected_gemv_bf16_bf16_out(                                                            \
      const uint16_t* x, const int64_t* selected, const uint8_t* qweight, uint16_t* out, int64_t x_rows,           \
      int64_t rows, int64_t num_experts, int64_t in_features, int64_t out_features, int64_t threads,               \
      hipengine_stream_t stream);                                                                                  \
  int hipengine_gguf_##q##_selected_silu_gemv_bf16_bf16_out(                                                       \
      const uint16_t* gate, const uint16_t* up, const int64_t* selected, const uint8_t* qweight, uint16_t* out,    \
      int64_t x_rows, int64_t rows, int64_t num_experts, int64_t in_features, int64_t out_features,                \
      int64_t threads, hipengine_stream_t stream);
HIPENGINE_GFX950_DECLARE_SELECTED_K(q5_k)
HIPENGINE_GFX950_DECLARE_SELECTED_K(q6_k)
HIPENGINE_GFX950_DECLARE_SELECTED_K(q8_0)

/* Decode gate/up pair: out[lane, n] = silu(bf16(gate)) * bf16(up), gate and up
 * rounded to bf16 before the activation as in gguf_q4_k_gemv.hip:732-736.
 * Replaces gguf_q4_k_gemv.hip:2751-2767. */
int hipengine_gguf_q4_k_selected_dual_silu_gemv_bf16_bf16_out(const uint16_t* x, const int64_t* selected,
                                                              const uint8_t* qweight_a, const uint8_t* qweight_b,
                                                              uint16_t* out, int64_t x_rows, int64_t rows,
                                                              int64_t num_experts, int64_t in_features,
                                                              int64_t out_features, int64_t threads,
                                                              hipengine_stream_t stream);

/* Decode gate/up pair without the activation: out_a[lane] = W_a[selected[lane]] . x_row,
 * out_b[lane] = W_b[selected[lane]] . x_row, one pass over both (the "dual" call kind,
 * loading/gguf_selected_contract.py:305-315).  Replaces gguf_q4_k_gemv.hip:2732-2749. */
int hipengine_gguf_q4_k_selected_dual_gemv_bf16_bf16_out(const uint16_t* x, const int64_t* selected,
                                                         const uint8_t* qweight_a, const uint8_t* qweight_b,
                                                         uint16_t* out_a, uint16_t* out_b, int64_t x_rows,
                                                         int64_t rows, int64_t num_experts, int64_t in_features,
                                                         int64_t out_features, int64_t threads,
                                                         hipengine_stream_t stream);

/* The same over pre-quantized activations: xq is [x_rows, in_features/32] 36-byte q8_1 blocks.
 * Replaces gguf_q4_k_gemv.hip:2864-2892. */
int hipengine_gguf_q4_k_selected_dual_gemv_q8_1_dp4a_bf16_bf16_out(const void* xq, const int64_t* selected,
                                                                   const uint8_t* qweight_a,
                                                                   const uint8_t* qweight_b, uint16_t* out_a,
                                                                   uint16_t* out_b, int64_t x_rows, int64_t rows,
                                                                   int64_t num_experts, int64_t in_features,
                                                                   int64_t out_features, int64_t threads,
                                                                   hipengine_stream_t stream);

/* Routed down projection with the weighted sum fused (the "weighted_down" call kind,
 * loading/gguf_selected_contract.py:50-54,305-315): x is [tokens*top_k, in_features] bf16, one row per lane;
 * out[t, :] = sum over the token's slots s = 0..top_k-1, in that order, of
 * routing_weights[t*top_k+s] * (W[selected[t*top_k+s]] . x[t*top_k+s]); lanes with an expert id outside
 * [0, num_experts) are skipped.  top_k <= 8, tokens*top_k <= 65535.  hipEngine has this call kind for its
 * IQ families only; the argument list is that of hipengine_gguf_iq4_xs_weighted_selected_down_bf16_bf16_out
 * (gguf_iq_gemv.hip:2276-2288). */
int hipengine_gguf_q4_k_weighted_selected_down_bf16_bf16_out(const uint16_t* x, const int64_t* selected,
                                                             const float* routing_weights, const uint8_t* qweight,
                                                             uint16_t* out, int64_t tokens, int64_t top_k,
                                                             int64_t num_experts, int64_t in_features,
                                                             int64_t out_features, int64_t threads,
                                                             hipengine_stream_t stream);
int hipengine_gguf_q6_k_weighted_selected_down_bf16_bf16_out(const uint16_t* x, const int64_t* selected,
                                                             const float* routing_weights, const uint8_t* qweight,
                                                             uint16_t* out, int64_t tokens, int64_t top_k,
                                                             int64_t num_experts, int64_t in_features,
                                                             int64_t out_features, int64_t threads,
                                                             hipengine_stream_t stream);

/* Grouped GEMV over gathered rows: x is [compact_rows, in_features] bf16 in expert-major order (the
 * packed_hidden of the routing index), rows [expert_start[e], expert_start[e+1]) belong to expert e and
 * out[r, :] = W[e] . x[r, :] for them; rows outside every range are left untouched.  An expert's weights
 * are read once per batch of 8 of its rows.  num_experts <= 65535.
 * Replaces gguf_q4_k_gemv.hip:2634-2669 (kernel :378-450; registry key
 * ("moe_linear", "gguf_q4_k", "selected_grouped_prefill_compact_rowbatch8_bf16_bf16_out"), gguf_q4_k_gemv.py:603-612). */
int hipengine_gguf_q4_k_selected_grouped_prefill_compact_rowbatch8_bf16_bf16_out(
    const void* x, const void* expert_start, const void* qweight, void* out, int64_t compact_rows,
    int64_t num_experts, int64_t in_features, int64_t out_features, hipengine_stream_t stream);

/* Grouped GEMV over gathered compact rows for expert weights of any of the four block types: rows
 * [expert_start[e], expert_start[e+1]) of x [compact_rows, in_features] (x_kind 0 f32, 1 bf16, 2 fp16, 3 q8_1
 * blocks) take expert e of qweight [num_experts, out_features, row_bytes]; out [compact_rows, out_features] of
 * out_kind.  An expert's weights are read once per 8 of its rows.  The form of
 * hipengine_gguf_q4_k_selected_grouped_prefill_compact_rowbatch8_bf16_bf16_out for Q5_K, Q6_K and Q8_0 experts
 * (the 35B-A3B shared expert is Q8_0) in the raw layout; hipEngine's grouped kernels for those types take its
 * RDNA3 layouts (t16 / pack8).  New here. */
int hipengine_gfx950_gguf_grouped_gemv(int32_t ggml_type, const void* x, int32_t x_kind, const int64_t* expert_start,
                                       const uint8_t* qweight, void* out, int32_t out_kind, int64_t compact_rows,
                                       int64_t num_experts, int64_t in_features, int64_t out_features,
                                       hipengine_stream_t stream);

/* The decode kernels with every choice explicit.  ggml_type 12 (Q4_K), 13 (Q5_K), 14 (Q6_K) or 8 (Q8_0); mode 1 takes
 * Q5_K and Q8_0 experts up to in_features 4096.
 *   mode 0: out[lanes, N] = W_a[selected[lane]] . x[lane / (lanes/x_rows)]
 *   mode 1: out[lanes, N] = silu(gate) * up with W_a = gate, W_b = up; round_mid != 0
 *           rounds gate and up to the output type first
 *   mode 2: x is [lanes, K] (one row per lane, lanes = x_rows * top_k); out[x_rows, N]
 *           = sum over the token's slots, in slot order, of routing_weights[lane] *
 *           (W_a[selected[lane]] . x[lane]); invalid experts are skipped; top_k <= 8
 * Kinds: 0 float32, 1 bf16, 2 fp16.  New here. */
int hipengine_gfx950_gguf_selected_gemv(int32_t ggml_type, int32_t mode, const void* x, int32_t x_kind,
                                        const int64_t* selected, const float* routing_weights,
                                        const uint8_t* qweight_a, const uint8_t* qweight_b, void* out,
                                        int32_t out_kind, int64_t x_rows, int64_t lanes, int64_t num_experts,
                                        int64_t top_k, int64_t in_features, int64_t out_features, int32_t round_mid,
                                        hipengine_stream_t stream);

/* Prefill: for every 32-row tile t with expert e = tile_expert[t] >= 0, the rows
 * r = expert_start_compact[e] + (32*t - expert_start_mmq32[e]) + 0..31 that lie
 * below expert_start_compact[e+1] get
 *   out[r, 0:Na]     = W_a[e] . x[compact_to_source[r]]
 *   out[r, Na:Na+Nb] = W_b[e] . x[compact_to_source[r]]
 * with x_q8 the DS4 blocks of the source rows.  expert_stride_rows is the
 * distance between experts in rows (0: the half's own width).  Na, Nb multiples
 * of 32, mmq_total_rows a multiple of 32 with at most 65535 tiles.
 * Replaces gguf_q4_k_q8_1_selected_prefill.hip:7426-7461 (body :1256-1670). */
int hipengine_gguf_q4_k_selected_dual_q8_1_ds4_mmq32_prefill_compact32_bf16_bf16_out(
    const void* x_q8, const int64_t* compact_to_source, const int64_t* expert_start_compact,
    const int64_t* expert_start_mmq32, const int64_t* tile_expert, const uint8_t* qweight_a,
    const uint8_t* qweight_b, uint16_t* out, int64_t compact_rows, int64_t in_features, int64_t out_features_a,
    int64_t out_features_b, int64_t num_experts, int64_t mmq_total_rows, int64_t expert_stride_rows,
    hipengine_stream_t stream);

/* hipEngine's 32 x 128 tile variant of the same GEMM (gguf_q4_k_q8_1_selected_prefill.hip:7510-7548): the same
 * arguments without the expert stride, the same results. */
int hipengine_gguf_q4_k_selected_dual_q8_1_ds4_mmq32x128_prefill_compact32_bf16_bf16_out(
    const void* x_q8, const int64_t* compact_to_source, const int64_t* expert_start_compact,
    const int64_t* expert_start_mmq32, const int64_t* tile_expert, const uint8_t* qweight_a, const uint8_t* qweight_b,
    uint16_t* out, int64_t compact_rows, int64_t in_features, int64_t out_features_a, int64_t out_features_b,
    int64_t num_experts, int64_t mmq_total_rows, hipengine_stream_t stream);

/* The same with the output kind explicit (0 float32, 1 bf16, 2 fp16), the source
 * row count given (indices are clamped to it), compact_to_source optional (NULL:
 * compact row r reads source row r) and the second weight optional
 * (out_features_b = 0).  New here. */
int hipengine_gfx950_gguf_q4_k_grouped_mmq(const void* x_q8, const int64_t* compact_to_source,
                                           const int64_t* expert_start_compact, const int64_t* expert_start_mmq32,
                                           const int64_t* tile_expert, const uint8_t* qweight_a,
                                           const uint8_t* qweight_b, void* out, int32_t out_kind,
                                           int64_t compact_rows, int64_t source_rows, int64_t in_features,
                                           int64_t out_features_a, int64_t out_features_b, int64_t num_experts,
                                           int64_t mmq_total_rows, int64_t expert_stride_rows,
                                           hipengine_stream_t stream);

/* hipengine_gfx950_gguf_q4_k_grouped_mmq for Q5_K expert weights [num_experts, out_features, K/256 * 176] over D4S4
 * activation blocks: the same arguments, tile map (32-row tiles) and limits; the arithmetic of
 * hipengine_gguf_q5_k_mmq32_q8_1_d4s4_f32_bf16_*_out per expert.  hipEngine has no grouped MMQ for Q5_K experts.
 * New here. */
int hipengine_gfx950_gguf_q5_k_grouped_mmq(const void* x_d4s4, const int64_t* compact_to_source,
                                           const int64_t* expert_start_compact, const int64_t* expert_start_mmq32,
                                           const int64_t* tile_expert, const uint8_t* qweight_a,
                                           const uint8_t* qweight_b, void* out, int32_t out_kind,
                                           int64_t compact_rows, int64_t source_rows, int64_t in_features,
                                           int64_t out_features_a, int64_t out_features_b, int64_t num_experts,
                                           int64_t mmq_total_rows, int64_t expert_stride_rows,
                                           hipengine_stream_t stream);

/* The expert-grouped MMQ for Q6_K expert weights [num_experts, out_features, K/256 * 210] over D4S4 activation
 * blocks (hipengine_gguf_q8_1_d4s4_f32_quantize_bf16 or hipengine_gfx950_moe_silu_mul_d4s4_pack):
 * out[compact row, :] = [W_a[e] | W_b[e]] x, e the expert that owns the compact row; the arithmetic of
 * hipengine_gguf_q6_k_mmq32_q8_1_d4s4_f32_bf16_*_out per expert.  The tile map is one of 128-row tiles
 * (hipengine_gfx950_moe_tile_map with tile_rows = 128): total_rows a multiple of 128 with at most 65535 tiles.
 * Any out_features; out_kind 0 float32, 1 bf16, 2 fp16; compact_to_source and the second weight optional.
 * hipEngine has no grouped MMQ for Q6_K experts (its grouped kernels for them take its RDNA3 layouts).  New here. */
int hipengine_gfx950_gguf_q6_k_grouped_mmq(const void* x_d4s4, const int64_t* compact_to_source,
                                           const int64_t* expert_start_compact, const int64_t* expert_start_tiles,
                                           const int64_t* tile_expert, const uint8_t* qweight_a,
                                           const uint8_t* qweight_b, void* out, int32_t out_kind,
                                           int64_t compact_rows, int64_t source_rows, int64_t in_features,
                                           int64_t out_features_a, int64_t out_features_b, int64_t num_experts,
                                           int64_t total_rows, int64_t expert_stride_rows,
                                           hipengine_stream_t stream);

/* hipengine_gfx950_gguf_q6_k_grouped_mmq for Q8_0 expert weights [num_experts, out_features, K/32 * 34]: the same
 * arguments, 128-row tile map and limits, in_features a multiple of 128; the arithmetic of
 * hipengine_gguf_q8_0_mmq32_q8_1_d4s4_f32_bf16_*_out per expert.  New here. */
int hipengine_gfx950_gguf_q8_0_grouped_mmq(const void* x_d4s4, const int64_t* compact_to_source,
                                           const int64_t* expert_start_compact, const int64_t* expert_start_tiles,
                                           const int64_t* tile_expert, const uint8_t* qweight_a,
                                           const uint8_t* qweight_b, void* out, int32_t out_kind,
                                           int64_t compact_rows, int64_t source_rows, int64_t in_features,
                                           int64_t out_features_a, int64_t out_features_b, int64_t num_experts,
                                           int64_t total_rows, int64_t expert_stride_rows,
                                           hipengine_stream_t stream);

/* hipengine_qwen35_moe_mmq32_tile_map for tiles of tile_rows = 32, 64 or 128 rows.  New here. */
int hipengine_gfx950_moe_tile_map(const int64_t* expert_start_compact, int64_t* tile_expert_start,
                                  int64_t* tile_expert, int64_t* total_out, int64_t num_experts,
                                  int64_t tile_capacity, int32_t tile_rows, hipengine_stream_t stream);

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

/* The same dots as the kernels that run on the int8 MFMA produce them: the production kernel body with one
 * more store per MFMA result.  form 3: the slab form (Q4_K), form 4: the phased slab form (Q4_K, Q5_K, Q6_K,
 * Q8_0), form 5: the direct slab form (Q4_K, Q6_K, Q8_0); all in their batch-8 instantiation, xq = 36-byte q8_1 blocks [rows, K/32], rows <= 8, shapes as
 * the forms take them.  dots as above; out: float32 [rows, out_features], the kernel's normal result. */
int hipengine_gfx950_gguf_gemv_mfma_dots_i32(int32_t ggml_type, int32_t form, const void* xq, const uint8_t* qweight,
                                             int32_t* dots, float* out, int64_t rows, int64_t in_features,
                                             int64_t out_features, hipengine_stream_t stream);

/* The same for the MMQ prefill GEMM: ggml_type 12 (Q4_K, xq = DS4 blocks, dots int32 [rows, N, K/32]), 13 (Q5_K,
 * xq = D4S4 blocks, dots [rows, N, K/32]), 14
 * (Q6_K, xq = D4S4 blocks, dots [rows, N, K/16], of the centred 6-bit values) or 8 (Q8_0, xq = D4S4 blocks, dots
 * [rows, N, K/32]); out: float32 [rows, N]. */
int hipengine_gfx950_gguf_mmq_dots_i32(int32_t ggml_type, const void* xq, const uint8_t* qweight, int32_t* dots,
                                       float* out, int64_t rows, int64_t in_features, int64_t out_features,
                                       hipengine_stream_t stream);

/* dst[0:bytes] = src[0:bytes] with a plain 16-byte-per-lane kernel (bytes % 16 == 0):
 * the known-size launch that HBM counter readings are calibrated against. */
int hipengine_gfx950_copy_bytes(const void* src, void* dst, int64_t bytes, hipengine_stream_t stream);

#ifdef __cplusplus
}
#endif

#endif /* HIPENGINE_GFX950_H */
