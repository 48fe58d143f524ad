/*
 * Tuning and measurement entry points of libhipengine_gfx950.so: the kernels of
 * hipengine_gfx950.h with their launch layout chosen by the caller, and host-only
 * queries of the layout the library would choose.  Parameter sweeps and benchmarks
 * use them; nothing in a serving path needs them and none has a counterpart in
 * hipEngine.  Same conventions as hipengine_gfx950.h (device pointers, int64 sizes,
 * hipError_t as int, asynchronous on `stream`).
 */
#ifndef HIPENGINE_GFX950_TUNING_H
#define HIPENGINE_GFX950_TUNING_H

#include "hipengine_gfx950.h"

#ifdef __cplusplus
extern "C" {
#endif

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

/* The same for the "stream" form (waves_total / waves workgroups of `waves` waves, all
 * resident; chunks of rows dealt round robin to the workgroups, groups of 16 blocks
 * round robin to a workgroup's waves, each wave keeping loads_in_flight loads in
 * flight; the library builds loads_in_flight = 2 only, deeper rings measured
 * slower).  rows <= 8, in_features >= 4096, at most one workgroup per chunk of
 * 16 / gcd(in_features / 256, 16) rows.  New here. */
int hipengine_gfx950_gguf_q8_1_fused_gemv_stream_tuned(int32_t ggml_type, const void* x, int32_t x_kind,
                                                       const uint8_t* qweight, void* out, int32_t out_kind,
                                                       int64_t rows, int64_t in_features, int64_t out_features,
                                                       int32_t loads_in_flight, int32_t waves, int32_t waves_total,
                                                       hipengine_stream_t stream);

/* The "slab" form for Q4_K: one workgroup per CU owns rows_per_workgroup (<= 96;
 * 0 = ceil(out_features / 256)) consecutive output rows, its waves split K in
 * slices of one or two 256-value blocks and run on the int8 MFMA.  rows <= 8,
 * 1024 <= in_features <= 6144.  New here. */
int hipengine_gfx950_gguf_q4_k_q8_1_fused_gemv_slab_tuned(const void* x, int32_t x_kind, const uint8_t* qweight,
                                                          void* out, int32_t out_kind, int64_t rows,
                                                          int64_t in_features, int64_t out_features,
                                                          int32_t rows_per_workgroup, hipengine_stream_t stream);

/* The phased slab form of the fused Q4_K / Q5_K / Q6_K / Q8_0 GEMV with an explicit layout
 * (0 = the planner's choice): `waves` <= 12 waves per workgroup split K by
 * 256-value blocks, `blocks_per_wave` (1, 2 or 4) per wave and phase, on the
 * int8 MFMA; `workgroups` share the output rows.  rows <= 8, in_features a
 * multiple of 512 and >= 2048, weights 4-byte aligned and < 4 GiB.  The default
 * dispatch uses this form for batches of 3 to 8 (Q4_K: where in_features > 6144,
 * below that its slab form).  New here. */
int hipengine_gfx950_gguf_q8_1_fused_gemv_pslab_tuned(int32_t ggml_type, const void* x, int32_t x_kind,
                                                      const uint8_t* qweight, void* out, int32_t out_kind,
                                                      int64_t rows, int64_t in_features, int64_t out_features,
                                                      int32_t waves, int32_t blocks_per_wave, int32_t workgroups,
                                                      hipengine_stream_t stream);

/* The direct slab form of the fused Q4_K / Q6_K / Q8_0 GEMV with an explicit layout (0 = the planner's
 * choice): weight blocks go from global memory straight into LDS (global_load_lds), `ring` steps of 16 rows
 * in flight per wave; `waves` <= 12 waves per workgroup split the K blocks of the workgroup's part, at most
 * two per wave; `k_parts` (1, 2, 4) splits K over workgroups, whose partial sums meet in a scratch array the
 * library holds (eight regions taken in turn by successive launches: more than eight such launches in flight at
 * once on one device share a region and race) and are added in part order by the workgroup that arrives last;
 * `workgroups` = row groups x k_parts.  rows <= 8, weights 2-byte aligned and < 4 GiB.  The default dispatch
 * takes this form for batches of 3 to 8 where K has to be split (in_features >= 6400 for Q4_K / Q6_K) and splits
 * into parts of equal length.  New here. */
int hipengine_gfx950_gguf_q8_1_fused_gemv_dslab_tuned(int32_t ggml_type, const void* x, int32_t x_kind,
                                                      const uint8_t* qweight, void* out, int32_t out_kind,
                                                      int64_t rows, int64_t in_features, int64_t out_features,
                                                      int32_t waves, int32_t ring, int32_t workgroups, int32_t k_parts,
                                                      hipengine_stream_t stream);

/* Host only: the layout the library picks for a shape, as
 * {batch_bucket, rows_per_lane, blocks_per_wave, k_slices, row_groups}.  New here. */
int hipengine_gfx950_gguf_gemv_default_plan(int32_t ggml_type, int64_t rows, int64_t in_features,
                                            int64_t out_features, int32_t* plan5);

/* Host only: the kernel form the default dispatch takes for the first launch of a
 * batch, as {form, rows in that launch}: form 0 row-strided, 1 run, 2 stream,
 * 3 slab (Q4_K on the int8 MFMA), 4 phased slab (int8 MFMA), 5 direct slab (int8 MFMA, weights
 * streamed straight into LDS, K split over workgroups).  Weights are assumed 4-byte aligned.  New here. */
int hipengine_gfx950_gguf_gemv_default_form(int32_t ggml_type, int64_t rows, int64_t in_features,
                                            int64_t out_features, int32_t* form2);

/* The same Q4_K x DS4 GEMM with the kernel form chosen by the caller (benchmarks
 * and tuning; no counterpart in hipEngine).  out_kind: 0 float32, 1 bf16, 2 fp16.
 * variant 0: the next K step is prefetched into registers (what the named entry
 * points run); variant 1: no prefetch, one more workgroup per CU. */
int hipengine_gfx950_gguf_q4_k_mmq_tuned(const void* xq, const uint8_t* qweight, void* out, int out_kind,
                                         int64_t rows, int64_t in_features, int64_t out_features, int variant,
                                         hipengine_stream_t stream);

/* Read-only pass over src[0 : bytes rounded down to 1 KB]: 256 workgroups of waves_per_workgroup resident waves,
 * each with loads_in_flight (2 or 4) wave-wide 16-byte-per-lane loads in flight, consecutive 1 KB pieces dealt
 * to consecutive waves.  Nothing is computed or written (sink, [256 * waves_per_workgroup] uint32 or null, is
 * there to keep the loads alive).  The time of this launch is what a decode GEMV over a weight of that size
 * could reach if its arithmetic, its activations and its stores were free.  src may be any even address: a base
 * that is 2 mod 4 shows what 16-byte loads from such addresses cost (every other 210-byte Q6_K block starts at one).
 * Measurement only.  New here. */
int hipengine_gfx950_read_probe(const void* src, int64_t bytes, int32_t waves_per_workgroup, int32_t loads_in_flight,
                                void* sink, hipengine_stream_t stream);

/* The same read-only pass over `workgroups` workgroups instead of one per CU (loads_in_flight 1, 2 or 4): with
 * thousands of workgroups every wave reads one or two pieces and leaves - the geometry of a launch that is
 * not persistent - so that the read ceilings quoted for this part do not rest on one launch shape.  Measurement
 * only.  New here. */
int hipengine_gfx950_read_probe_grid(const void* src, int64_t bytes, int32_t waves_per_workgroup, int32_t loads_in_flight,
                                     int32_t workgroups, void* sink, hipengine_stream_t stream);

#ifdef __cplusplus
}
#endif

#endif /* HIPENGINE_GFX950_TUNING_H */
