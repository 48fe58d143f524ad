// Verification exports: the block unpack and the int32 sub-block dots of the
// production kernels, written to memory so a CPU oracle can compare them bit
// for bit.  Both kernels call the same device functions as the GEMV
// (gguf_common.hpp unpack, gemv_load_block / gemv_block_dots).

#include "gguf_gemv.hpp"

#include "../../include/hipengine_gfx950.h"

namespace {

using namespace hipengine_gfx950;

__device__ __forceinline__ float byte_f(uint32_t w, int i) { return static_cast<float>((w >> (8 * i)) & 0xFFu); }

// One thread per qs dword: 32 threads per Q4_K block.
__global__ void __launch_bounds__(256) dequant_q4_k_kernel(const uint8_t* __restrict__ blocks, float* __restrict__ out,
                                                           int64_t n_blocks) {
  const int64_t t = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  const int64_t b = t >> 5;
  if (b >= n_blocks) return;
  const int i = static_cast<int>(t & 31);
  const uint8_t* blk = blocks + b * Q4_K_BYTES;
  const uint4 h = load16(blk);
  const uint32_t qs = load4(blk + 16 + 4 * i);
  const Q4KScales s = q4k_unpack_scales(h.y, h.z, h.w);
  const float d = f16_bits_to_float(h.x & 0xFFFFu), dmin = f16_bits_to_float(h.x >> 16);
  const int pair = i >> 3, lane0 = (i & 7) * 4;
  const float sa = d * static_cast<float>(q4k_scale_of(s, 2 * pair));
  const float sb = d * static_cast<float>(q4k_scale_of(s, 2 * pair + 1));
  const float ma = dmin * static_cast<float>(q4k_min_of(s, 2 * pair));
  const float mb = dmin * static_cast<float>(q4k_min_of(s, 2 * pair + 1));
  const uint32_t lo = q4k_low(qs), hi = q4k_high(qs);
  float* o = out + b * QK_K;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    o[(2 * pair) * 32 + lane0 + j] = sa * byte_f(lo, j) - ma;
    o[(2 * pair + 1) * 32 + lane0 + j] = sb * byte_f(hi, j) - mb;
  }
}

// One thread per (half, lane dword): 16 threads per Q6_K block.
__global__ void __launch_bounds__(256) dequant_q6_k_kernel(const uint8_t* __restrict__ blocks, float* __restrict__ out,
                                                           int64_t n_blocks) {
  const int64_t t = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  const int64_t b = t >> 4;
  if (b >= n_blocks) return;
  const int h = static_cast<int>(t >> 3) & 1, i = static_cast<int>(t & 7);
  const uint8_t* blk = blocks + b * Q6_K_BYTES;
  const Q6KQuad u = q6k_unpack(load4(blk + 64 * h + 4 * i), load4(blk + 64 * h + 32 + 4 * i),
                               load4(blk + 128 + 32 * h + 4 * i));
  const uint32_t g[4] = {q6k_center(u.g0), q6k_center(u.g1), q6k_center(u.g2), q6k_center(u.g3)};
  const float d = f16_bits_to_float(load2(blk + 208));
  const int8_t* sc = reinterpret_cast<const int8_t*>(blk + 192);
  float* o = out + b * QK_K;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int grp = 4 * h + j;
    const float step = d * static_cast<float>(sc[grp * 2 + (i >> 2)]);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int q = static_cast<int8_t>((g[j] >> (8 * e)) & 0xFFu);
      o[grp * 32 + 4 * i + e] = step * static_cast<float>(q);
    }
  }
}

// One thread per quant dword: 8 threads per Q8_0 block.
__global__ void __launch_bounds__(256) dequant_q8_0_kernel(const uint8_t* __restrict__ blocks, float* __restrict__ out,
                                                           int64_t n_blocks) {
  const int64_t t = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  const int64_t b = t >> 3;
  if (b >= n_blocks) return;
  const int i = static_cast<int>(t & 7);
  const uint8_t* blk = blocks + b * Q8_0_BYTES;
  const float d = f16_bits_to_float(load2(blk));
  const uint32_t w = (load2(blk + 2 + 4 * i)) | (load2(blk + 4 + 4 * i) << 16);
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    out[b * 32 + 4 * i + e] = static_cast<float>(static_cast<int8_t>((w >> (8 * e)) & 0xFFu)) * d;
  }
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

}  // namespace

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
  const int per_block = ggml_type == GGML_Q4_K ? 32 : ggml_type == GGML_Q6_K ? 16 : ggml_type == GGML_Q8_0 ? 8 : 0;
  if (!per_block) return static_cast<int>(hipErrorInvalidValue);
  const int64_t grid = (n_blocks * per_block + 255) / 256;
  if (grid > 0x7FFFFFFF) return static_cast<int>(hipErrorInvalidValue);
  const dim3 g(static_cast<unsigned>(grid)), b(256);
  if (ggml_type == GGML_Q4_K) hipLaunchKernelGGL(dequant_q4_k_kernel, g, b, 0, stream, blocks, out, n_blocks);
  else if (ggml_type == GGML_Q6_K) hipLaunchKernelGGL(dequant_q6_k_kernel, g, b, 0, stream, blocks, out, n_blocks);
  else hipLaunchKernelGGL(dequant_q8_0_kernel, g, b, 0, stream, blocks, out, n_blocks);
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
  } else if (ggml_type == GGML_Q6_K) {
    hipLaunchKernelGGL(block_dots_kernel<GGML_Q6_K>, g, dim3(64), 0, stream, x, qweight, dots, qsums, K, N);
  } else if (ggml_type == GGML_Q8_0) {
    hipLaunchKernelGGL(block_dots_kernel<GGML_Q8_0>, g, dim3(64), 0, stream, x, qweight, dots, qsums, K, N);
  } else {
    return static_cast<int>(hipErrorInvalidValue);
  }
  return static_cast<int>(hipGetLastError());
}
