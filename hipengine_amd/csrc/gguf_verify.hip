// Verification exports: the block unpack and the int32 sub-block dots of the
// production kernels, written to memory so a CPU oracle can compare them bit
// for bit.  Both kernels call the same device functions as the GEMV
// (gguf_common.hpp unpack, gemv_load_block / gemv_block_dots).

#include "gguf_gemv.hpp"
#include "gguf_dequant.hpp"

#include "../../include/hipengine_gfx950.h"

namespace {

using namespace hipengine_gfx950;

// One unit of a block per thread (gguf_dequant.hpp).
template <int QT>
__global__ void __launch_bounds__(256) dequant_kernel(const uint8_t* __restrict__ blocks, float* __restrict__ out,
                                                      int64_t n_blocks) {
  using T = DequantTraits<QT>;
  const int64_t t = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  const int64_t b = t / T::UNITS;
  if (b >= n_blocks) return;
  float* o = out + b * T::VALUES;
  dequant_unit<QT>(blocks + b * T::BYTES, static_cast<int>(t - b * T::UNITS), [=](int k, float v) { o[k] = v; });
}

// One wave per (16 weight rows, one 256-value K block); grid (ceil(N/16), K/256, rows).
template <int QT>
__global__ void __launch_bounds__(64) block_dots_kernel(const uint8_t* __restrict__ xq, const uint8_t* __restrict__ w,
                                                        int32_t* __restrict__ dots, int32_t* __restrict__ qsums,
                                                        int K, int N) {
  __shared__ __align__(16) uint8_t q8[QK_K];
  __shared__ int s16[16];
  const int lane = threadIdx.x, q = lane & 3, rg = lane >> 2;
  const int kb = blockIdx.y, brow = blockIdx.z;
  const int nsb = K / 32;
  // stage the 8 q8_1 blocks of this K block: lane -> (block lane>>3, dword lane&7)
  {
    const uint8_t* blk = xq + (static_cast<int64_t>(brow) * nsb + kb * 8 + (lane >> 3)) * Q8_1_BYTES;
    const uint32_t packed = *reinterpret_cast<const uint32_t*>(blk + 4 + 4 * (lane & 7));
    *reinterpret_cast<uint32_t*>(q8 + lane * 4) = packed;
    int part = dot4(0x01010101u, packed, 0);
    part += dpp_i<DPP_QUAD_XOR1>(part);
    part += dpp_i<DPP_QUAD_XOR2>(part);
    if ((lane & 3) == 0) s16[lane >> 2] = part;
  }
  __syncthreads();
  if (qsums != nullptr && blockIdx.x == 0 && lane < 8) {
    qsums[static_cast<int64_t>(brow) * nsb + kb * 8 + lane] = s16[2 * lane] + s16[2 * lane + 1];
  }
  const int row = blockIdx.x * 16 + rg;
  if (row >= N) return;
  const int64_t row_bytes = static_cast<int64_t>(K / QK_K) * GemvTraits<QT>::SUPER_BYTES;
  WeightRegs<GemvTraits<QT>::REGS> r;
  gemv_load_block<QT>(w + row * row_bytes + static_cast<int64_t>(kb) * GemvTraits<QT>::SUPER_BYTES, q, r);
  int d[4];
  gemv_block_dots<QT>(r, q, q8, s16, d);
  if constexpr (QT == GGML_Q6_K) {
    int32_t* o = dots + (static_cast<int64_t>(brow) * N + row) * (K / 16) + kb * 16;
    const int h = q >> 1, t = q & 1;
#pragma unroll
    for (int j = 0; j < 4; ++j) o[(4 * h + j) * 2 + t] = d[j];
  } else {
    int32_t* o = dots + (static_cast<int64_t>(brow) * N + row) * nsb + kb * 8;
    o[2 * q] = d[0];
    o[2 * q + 1] = d[1];
  }
}

// Plain 16-byte-per-lane copy: the known-size kernel that hardware counter
// readings (HBM fetch / write sizes) are calibrated against.
__global__ void __launch_bounds__(256) copy_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst, int64_t n16) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n16; i += stride) dst[i] = src[i];
}

// Read-only pass over a buffer with the streaming GEMV's load shape: resident waves, each with DEPTH wave-wide
// 16-byte-per-lane loads (1 KB) in flight, consecutive pieces dealt to consecutive waves of the whole grid.
// What a launch that only reads can reach; nothing is computed, and the store never happens for real data
// (it keeps the loads from being dropped).
template <int DEPTH>
__global__ void __launch_bounds__(1024) read_probe_kernel(const uint4* __restrict__ src, int64_t pieces, int rounds,
                                                          uint32_t* __restrict__ sink) {
  const int lane = threadIdx.x & 63;
  const int64_t waves_total = static_cast<int64_t>(gridDim.x) * (blockDim.x >> 6);
  const int64_t gw = static_cast<int64_t>(blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6);
  uint4 ring[DEPTH];
  uint32_t acc = 0;
  auto piece = [&](int i) {                       // rounds past the end re-read the last piece
    const int64_t p = static_cast<int64_t>(i) * waves_total + gw;
    return src[(p < pieces ? p : pieces - 1) * 64 + lane];
  };
#pragma unroll
  for (int c = 0; c < DEPTH; ++c) ring[c] = piece(c);
  for (int i0 = 0; i0 < rounds; i0 += DEPTH) {
#pragma unroll
    for (int c = 0; c < DEPTH; ++c) {
      acc ^= ring[c].x ^ ring[c].y ^ ring[c].z ^ ring[c].w;
      ring[c] = piece(i0 + c + DEPTH);
    }
  }
#pragma unroll
  for (int c = 0; c < DEPTH; ++c) acc ^= ring[c].x;
  if (acc == 0x9E3779B9u && sink) sink[gw] = acc;
}

}  // namespace

static int read_probe_launch(const void* src, int64_t bytes, int32_t waves_per_workgroup, int32_t loads_in_flight,
                             int32_t workgroups, void* sink, hipStream_t stream);

extern "C" int hipengine_gfx950_read_probe(const void* src, int64_t bytes, int32_t waves_per_workgroup,
                                           int32_t loads_in_flight, void* sink, hipStream_t stream) {
  if (loads_in_flight == 1) return static_cast<int>(hipErrorInvalidValue);
  return read_probe_launch(src, bytes, waves_per_workgroup, loads_in_flight, 256, sink, stream);
}

// The same probe over `workgroups` workgroups instead of one per CU: with thousands of them a wave reads one or
// two pieces and leaves, the geometry of a launch that is not persistent.  loads_in_flight may be 1 here.
extern "C" int hipengine_gfx950_read_probe_grid(const void* src, int64_t bytes, int32_t waves_per_workgroup,
                                                int32_t loads_in_flight, int32_t workgroups, void* sink,
                                                hipStream_t stream) {
  if (workgroups < 1 || workgroups > (1 << 20)) return static_cast<int>(hipErrorInvalidValue);
  return read_probe_launch(src, bytes, waves_per_workgroup, loads_in_flight, workgroups, sink, stream);
}

static int read_probe_launch(const void* src, int64_t bytes, int32_t waves_per_workgroup, int32_t loads_in_flight,
                             int32_t workgroups, void* sink, hipStream_t stream) {
  if (!src || (reinterpret_cast<uintptr_t>(src) & 1) != 0 || bytes < 1024 || waves_per_workgroup < 1 || waves_per_workgroup > 16 ||
      (loads_in_flight != 1 && loads_in_flight != 2 && loads_in_flight != 4)) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  const int64_t pieces = bytes / 1024;            // whole 1 KB pieces: every load stays inside [src, src + bytes)
  const int grid = workgroups;
  const int64_t waves_total = static_cast<int64_t>(grid) * waves_per_workgroup;
  const int64_t rounds64 = (pieces + waves_total - 1) / waves_total;
  if (rounds64 > (1 << 28)) return static_cast<int>(hipErrorInvalidValue);
  const int rounds = static_cast<int>(rounds64);
  if (loads_in_flight == 1) {
    hipLaunchKernelGGL(read_probe_kernel<1>, dim3(grid), dim3(waves_per_workgroup * 64), 0, stream,
                       static_cast<const uint4*>(src), pieces, rounds, static_cast<uint32_t*>(sink));
  } else if (loads_in_flight == 2) {
    hipLaunchKernelGGL(read_probe_kernel<2>, dim3(grid), dim3(waves_per_workgroup * 64), 0, stream,
                       static_cast<const uint4*>(src), pieces, rounds, static_cast<uint32_t*>(sink));
  } else {
    hipLaunchKernelGGL(read_probe_kernel<4>, dim3(grid), dim3(waves_per_workgroup * 64), 0, stream,
                       static_cast<const uint4*>(src), pieces, rounds, static_cast<uint32_t*>(sink));
  }
  return static_cast<int>(hipGetLastError());
}

extern "C" int hipengine_gfx950_copy_bytes(const void* src, void* dst, int64_t bytes, hipStream_t stream) {
  if (!src || !dst || bytes <= 0 || (bytes % 16) != 0) return static_cast<int>(hipErrorInvalidValue);
  const int64_t n16 = bytes / 16;
  const int64_t want = (n16 + 255) / 256;
  hipLaunchKernelGGL(copy_kernel, dim3(static_cast<unsigned>(want < 16384 ? want : 16384)), dim3(256), 0, stream,
                     static_cast<const uint4*>(src), static_cast<uint4*>(dst), n16);
  return static_cast<int>(hipGetLastError());
}

extern "C" int hipengine_gfx950_gguf_dequantize_f32(int32_t ggml_type, const uint8_t* blocks, float* out,
                                                    int64_t n_blocks, hipStream_t stream) {
  if (!blocks || !out || n_blocks <= 0) return static_cast<int>(hipErrorInvalidValue);
  const int per_block = ggml_type == GGML_Q4_K || ggml_type == GGML_Q5_K ? 32
                        : ggml_type == GGML_Q6_K ? 16 : ggml_type == GGML_Q8_0 ? 8 : 0;
  if (!per_block) return static_cast<int>(hipErrorInvalidValue);
  const int64_t grid = (n_blocks * per_block + 255) / 256;
  if (grid > 0x7FFFFFFF) return static_cast<int>(hipErrorInvalidValue);
  const dim3 g(static_cast<unsigned>(grid)), b(256);
  if (ggml_type == GGML_Q4_K) hipLaunchKernelGGL(dequant_kernel<GGML_Q4_K>, g, b, 0, stream, blocks, out, n_blocks);
  else if (ggml_type == GGML_Q5_K) hipLaunchKernelGGL(dequant_kernel<GGML_Q5_K>, g, b, 0, stream, blocks, out, n_blocks);
  else if (ggml_type == GGML_Q6_K) hipLaunchKernelGGL(dequant_kernel<GGML_Q6_K>, g, b, 0, stream, blocks, out, n_blocks);
  else hipLaunchKernelGGL(dequant_kernel<GGML_Q8_0>, g, b, 0, stream, blocks, out, n_blocks);
  return static_cast<int>(hipGetLastError());
}

extern "C" int hipengine_gfx950_gguf_q8_1_block_dots_i32(int32_t ggml_type, const void* xq, const uint8_t* qweight,
                                                         int32_t* dots, int32_t* qsums, int64_t rows,
                                                         int64_t in_features, int64_t out_features,
                                                         hipStream_t stream) {
  if (!xq || !qweight || !dots || rows <= 0 || rows > 65535 || in_features <= 0 || (in_features % QK_K) != 0 ||
      in_features / QK_K > 65535 || out_features <= 0 || out_features > (1 << 30)) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  const dim3 g(static_cast<unsigned>((out_features + 15) / 16), static_cast<unsigned>(in_features / QK_K),
               static_cast<unsigned>(rows));
  const uint8_t* x = static_cast<const uint8_t*>(xq);
  const int K = static_cast<int>(in_features), N = static_cast<int>(out_features);
  if (ggml_type == GGML_Q4_K) {
    hipLaunchKernelGGL(block_dots_kernel<GGML_Q4_K>, g, dim3(64), 0, stream, x, qweight, dots, qsums, K, N);
  } else if (ggml_type == GGML_Q5_K) {
    hipLaunchKernelGGL(block_dots_kernel<GGML_Q5_K>, g, dim3(64), 0, stream, x, qweight, dots, qsums, K, N);
  } else if (ggml_type == GGML_Q6_K) {
    hipLaunchKernelGGL(block_dots_kernel<GGML_Q6_K>, g, dim3(64), 0, stream, x, qweight, dots, qsums, K, N);
  } else if (ggml_type == GGML_Q8_0) {
    hipLaunchKernelGGL(block_dots_kernel<GGML_Q8_0>, g, dim3(64), 0, stream, x, qweight, dots, qsums, K, N);
  } else {
    return static_cast<int>(hipErrorInvalidValue);
  }
  return static_cast<int>(hipGetLastError());
}
