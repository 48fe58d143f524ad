// Per-device set-up steps of the library, collected by hipengine_gfx950_init() (gguf_init.hip).
// Each returns a hipError_t as int and may be called again for a device already set up.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace hipengine_gfx950 {

// Raise the dynamic-LDS limit of every decode GEMV kernel that may be launched with more than 64 KB
// (gguf_gemv.hip).  Applies to the current device.
int gemv_raise_lds_limits();

// Look up this device's address of the arg-max stage scratch (gguf_argmax.hip).  `device` must be current.
int argmax_noalloc_setup(int device);

// Look up this device's address of the pack buffer of the dense prefill entries (gguf_mmq.hip).
int prefill_pack_setup(int device);

// Dense prefill from bf16 activations through the pack buffer the library holds (gguf_mmq.hip): whether a shape
// goes that way (32 rows or more, a shape the MMQ of the type takes, at least 128 packed rows fit the buffer),
// and the call itself: chunks of up to 512 rows, pack then MMQ, nothing allocated.
bool prefill_library_buffer_takes(int ggml_type, int64_t rows, int64_t in_features, int64_t out_features);
int prefill_bf16_library_buffer(int ggml_type, const void* x, const uint8_t* qweight, void* out, int out_kind, int64_t rows,
                                int64_t in_features, int64_t out_features, hipStream_t stream);

// Make the runtime load the code object of a source file now (it otherwise does so at the file's first
// launch, which may be inside a stream capture): one per source file that has kernels and no other set-up.
int quantize_load();
int mmq_load();
int moe_load();
int embedding_load();

// True once hipengine_gfx950_init() has completed for the current device; runs it otherwise.
// Launch paths that depend on the set-up call this first.
int ensure_init();

}  // namespace hipengine_gfx950
