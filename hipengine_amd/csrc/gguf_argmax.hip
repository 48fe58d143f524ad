// Row-wise arg-max of float32 logits (the step after the lm_head GEMV of a greedy decode):
// highest value, lowest index among equals.  Two stages over caller-owned scratch, laid out
// exactly as hipEngine's hipengine_argmax_f32_rows_i32 uses it
// (kernels/hip_gfx1100/linear/lm_head.hip:286-365,746-793): stage 1 writes one (value, index)
// pair per block of threads*4 logits into block_values / block_indices [rows, stage1_blocks],
// stage 2 reduces a row's pairs.

#include "gguf_common.hpp"
#include "gguf_init.hpp"

#include <atomic>
#include <mutex>

#include "../../include/hipengine_gfx950.h"

namespace {

using namespace hipengine_gfx950;

constexpr float ARGMAX_LOWEST = -3.4028234663852886e+38F;

__device__ __forceinline__ bool better_pair(float v, int i, float bv, int bi) { return v > bv || (v == bv && i < bi); }

// Best pair of the workgroup (<= 16 waves), valid in thread 0.
__device__ __forceinline__ void block_best(float& v, int& i, float* sv, int* si) {
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const float ov = __shfl_xor(v, off);
    const int oi = __shfl_xor(i, off);
    if (better_pair(ov, oi, v, i)) { v = ov; i = oi; }
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = (blockDim.x + 63) >> 6;
  if (lane == 0) { sv[wave] = v; si[wave] = i; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < waves; ++w)
      if (better_pair(sv[w], si[w], v, i)) { v = sv[w]; i = si[w]; }
  }
}

__global__ void __launch_bounds__(512) argmax_stage1_kernel(const float* __restrict__ logits, float* __restrict__ block_values,
                                                            int32_t* __restrict__ block_indices, int64_t vocab_size,
                                                            int64_t stage1_blocks) {
  __shared__ float sv[16];
  __shared__ int si[16];
  const int64_t row = blockIdx.y;
  const int64_t begin = static_cast<int64_t>(blockIdx.x) * blockDim.x * 4;
  const int64_t end = min(begin + static_cast<int64_t>(blockDim.x) * 4, vocab_size);
  const float* src = logits + row * vocab_size;
  float v = ARGMAX_LOWEST;
  int i = 0x7FFFFFFF;
  for (int64_t k = begin + threadIdx.x; k < end; k += blockDim.x) {
    const float x = src[k];
    if (better_pair(x, static_cast<int>(k), v, i)) { v = x; i = static_cast<int>(k); }
  }
  block_best(v, i, sv, si);
  if (threadIdx.x == 0) {
    block_values[row * stage1_blocks + blockIdx.x] = v;
    block_indices[row * stage1_blocks + blockIdx.x] = i;
  }
}

__global__ void __launch_bounds__(512) argmax_stage2_kernel(const float* __restrict__ block_values,
                                                            const int32_t* __restrict__ block_indices,
                                                            int32_t* __restrict__ out_indices, float* __restrict__ out_values,
                                                            int64_t num_blocks) {
  __shared__ float sv[16];
  __shared__ int si[16];
  const int64_t row = blockIdx.x;
  float v = ARGMAX_LOWEST;
  int i = 0x7FFFFFFF;
  for (int64_t k = threadIdx.x; k < num_blocks; k += blockDim.x) {
    const float x = block_values[row * num_blocks + k];
    const int xi = block_indices[row * num_blocks + k];
    if (better_pair(x, xi, v, i)) { v = x; i = xi; }
  }
  block_best(v, i, sv, si);
  if (threadIdx.x == 0) {
    out_indices[row] = i;
    if (out_values) out_values[row] = v;
  }
}

// ---- stage scratch held by the library, for callers that cannot allocate ----
//
// One (value, index) pair per stage-1 block, HIPENGINE_GFX950_ARGMAX_NOALLOC_MAX_ENTRIES pairs at most:
// values in the first half of the array, indices in the second.  Every device the library runs on holds
// its own copy of the array at its own address until the process ends; `scratch` is only a host-side
// handle, the address kernels may use is the one hipGetSymbolAddress returns with that device current.
constexpr int64_t kNoAllocEntries = HIPENGINE_GFX950_ARGMAX_NOALLOC_MAX_ENTRIES;
static __device__ __align__(256) uint8_t scratch[kNoAllocEntries * (sizeof(float) + sizeof(int32_t))];

constexpr int kMaxDevices = 64;
std::mutex scratch_mutex;
std::atomic<void*> scratch_ptr[kMaxDevices];   // per device, null until set up

}  // namespace

namespace hipengine_gfx950 {

int argmax_noalloc_setup(int device) {
  if (device < 0 || device >= kMaxDevices) return static_cast<int>(hipErrorInvalidDevice);
  std::lock_guard<std::mutex> lock(scratch_mutex);
  if (scratch_ptr[device].load(std::memory_order_acquire)) return static_cast<int>(hipSuccess);
  void* ptr = nullptr;
  const hipError_t err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
  if (err != hipSuccess) return static_cast<int>(err);
  if (!ptr) return static_cast<int>(hipErrorInvalidSymbol);
  scratch_ptr[device].store(ptr, std::memory_order_release);
  return static_cast<int>(hipSuccess);
}

}  // namespace hipengine_gfx950

namespace {

int launch_argmax(const float* logits, float* block_values, int32_t* block_indices, int32_t* out_indices,
                  float* out_values, int64_t rows, int64_t vocab_size, int64_t threads, int64_t stage1_blocks,
                  hipStream_t stream) {
  const unsigned t = static_cast<unsigned>(threads);
  hipLaunchKernelGGL(argmax_stage1_kernel, dim3(static_cast<unsigned>(stage1_blocks), static_cast<unsigned>(rows)),
                     dim3(t), 0, stream, logits, block_values, block_indices, vocab_size, stage1_blocks);
  const hipError_t err = hipGetLastError();
  if (err != hipSuccess) return static_cast<int>(err);
  hipLaunchKernelGGL(argmax_stage2_kernel, dim3(static_cast<unsigned>(rows)), dim3(t), 0, stream, block_values,
                     block_indices, out_indices, out_values, stage1_blocks);
  return static_cast<int>(hipGetLastError());
}

}  // namespace

extern "C" int hipengine_gfx950_argmax_f32_rows_i32_noalloc(const float* logits, int32_t* out_indices,
                                                            float* out_values, int64_t rows, int64_t vocab_size,
                                                            int64_t threads, hipStream_t stream) {
  if (!logits || !out_indices || rows <= 0 || rows > 65535 || vocab_size <= 0 || vocab_size > 0x7FFFFFFF ||
      !(threads == 128 || threads == 256 || threads == 512)) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  const int64_t stage1_blocks = (vocab_size + threads * 4 - 1) / (threads * 4);
  if (rows * stage1_blocks > kNoAllocEntries) return static_cast<int>(hipErrorInvalidValue);   // beyond the array
  int device = -1;
  hipError_t err = hipGetDevice(&device);
  if (err != hipSuccess) return static_cast<int>(err);
  if (device < 0 || device >= kMaxDevices) return static_cast<int>(hipErrorInvalidDevice);
  if (!scratch_ptr[device].load(std::memory_order_acquire)) {   // first call on this device without hipengine_gfx950_init()
    const int rc = hipengine_gfx950::argmax_noalloc_setup(device);
    if (rc != static_cast<int>(hipSuccess)) return rc;
  }
  // Stage 1 writes every pair stage 2 reads, so nothing of the previous call's contents is consumed.
  uint8_t* base = static_cast<uint8_t*>(scratch_ptr[device].load(std::memory_order_acquire));
  float* block_values = reinterpret_cast<float*>(base);
  int32_t* block_indices = reinterpret_cast<int32_t*>(base + kNoAllocEntries * sizeof(float));
  return launch_argmax(logits, block_values, block_indices, out_indices, out_values, rows, vocab_size, threads,
                       stage1_blocks, stream);
}

extern "C" int hipengine_argmax_f32_rows_i32(const float* logits, float* block_values, int32_t* block_indices,
                                             int32_t* out_indices, float* out_values, int64_t rows, int64_t vocab_size,
                                             int64_t threads, hipStream_t stream) {
  if (!logits || !block_values || !block_indices || !out_indices || rows <= 0 || rows > 65535 || vocab_size <= 0 ||
      vocab_size > 0x7FFFFFFF || !(threads == 128 || threads == 256 || threads == 512)) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  const int64_t stage1_blocks = (vocab_size + threads * 4 - 1) / (threads * 4);
  return launch_argmax(logits, block_values, block_indices, out_indices, out_values, rows, vocab_size, threads,
                       stage1_blocks, stream);
}
