// Stand-alone q8_1 activation quantizers for gfx950: the 36-byte GEMV
// convention, the 144-byte DS4 (MMQ) convention and the 160-byte D4S4 one.
// Eight lanes share a 32-value group (four consecutive values per lane, one
// 16-byte or 8-byte load), so a wave covers eight groups per pass and the
// group reductions are DPP only.

#include "gguf_common.hpp"

#include "gguf_init.hpp"

#include "../../include/hipengine_gfx950.h"

namespace {

using namespace hipengine_gfx950;

__device__ __forceinline__ void load4_values(const void* x, int kind, int64_t idx, float (&v)[4]) {
  if (kind == KIND_F32) {
    const float4 t = *reinterpret_cast<const float4*>(static_cast<const float*>(x) + idx);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
  } else {
    const uint2 t = *reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(x) + idx);
    if (kind == KIND_BF16) {
      v[0] = bf16_bits_to_float(t.x & 0xFFFFu); v[1] = bf16_bits_to_float(t.x >> 16);
      v[2] = bf16_bits_to_float(t.y & 0xFFFFu); v[3] = bf16_bits_to_float(t.y >> 16);
    } else {
      v[0] = f16_bits_to_float(t.x & 0xFFFFu); v[1] = f16_bits_to_float(t.x >> 16);
      v[2] = f16_bits_to_float(t.y & 0xFFFFu); v[3] = f16_bits_to_float(t.y >> 16);
    }
  }
}

__device__ __forceinline__ uint32_t pack_i8x4(int a, int b, int c, int d) {
  return (a & 0xFF) | ((b & 0xFF) << 8) | ((c & 0xFF) << 16) | (static_cast<uint32_t>(d & 0xFF) << 24);
}

// 36-byte blocks.  Grid: x = ceil(groups / 32), 256 threads = 32 groups.
__global__ void __launch_bounds__(256) quantize_q8_1_kernel(const void* __restrict__ x, int kind,
                                                            uint8_t* __restrict__ xq, int64_t total_groups) {
  const int64_t g = static_cast<int64_t>(blockIdx.x) * 32 + (threadIdx.x >> 3);
  const int e = threadIdx.x & 7;
  if (g >= total_groups) return;   // uniform for the 8 lanes of a group
  float v[4];
  load4_values(x, kind, g * 32 + e * 4, v);
  const float amax = oct_max(fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3]))));
  const float sum = oct_tree_sum32(v[0], v[1], v[2], v[3]);
  const float d = amax / 127.0f;
  uint32_t packed = 0;
  if (amax != 0.0f) {
    packed = pack_i8x4(max(-128, min(127, static_cast<int>(roundf(v[0] / d)))),
                       max(-128, min(127, static_cast<int>(roundf(v[1] / d)))),
                       max(-128, min(127, static_cast<int>(roundf(v[2] / d)))),
                       max(-128, min(127, static_cast<int>(roundf(v[3] / d)))));
  }
  uint8_t* blk = xq + g * Q8_1_BYTES;
  *reinterpret_cast<uint32_t*>(blk + 4 + 4 * e) = packed;
  if (e == 0) {
    *reinterpret_cast<uint32_t*>(blk) =
        static_cast<uint32_t>(float_to_f16_bits(d)) | (static_cast<uint32_t>(float_to_f16_bits(sum)) << 16);
  }
}

// Two planes of 36-byte blocks (gguf_q4_k_gemv.hip:777-829): plane 0 is the plain quantization, plane 1, at
// +total_groups blocks, the same quantization of what plane 0 leaves, x - float(half d0) * q0 (the product has 19
// significant bits, so the subtraction is one rounding however it is contracted).
__global__ void __launch_bounds__(256) quantize_q8_1x2_kernel(const void* __restrict__ x, int kind,
                                                              uint8_t* __restrict__ xq, int64_t total_groups) {
  const int64_t g = static_cast<int64_t>(blockIdx.x) * 32 + (threadIdx.x >> 3);
  const int e = threadIdx.x & 7;
  if (g >= total_groups) return;   // uniform for the 8 lanes of a group
  float v[4];
  load4_values(x, kind, g * 32 + e * 4, v);
#pragma unroll
  for (int plane = 0; plane < 2; ++plane) {
    const float amax = oct_max(fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3]))));
    const float sum = oct_tree_sum32(v[0], v[1], v[2], v[3]);
    const float d = amax / 127.0f;
    int q[4] = {0, 0, 0, 0};
    if (amax != 0.0f) {
#pragma unroll
      for (int i = 0; i < 4; ++i) q[i] = max(-128, min(127, static_cast<int>(roundf(v[i] / d))));
    }
    uint8_t* blk = xq + (plane * total_groups + g) * Q8_1_BYTES;
    *reinterpret_cast<uint32_t*>(blk + 4 + 4 * e) = pack_i8x4(q[0], q[1], q[2], q[3]);
    const uint16_t dh = float_to_f16_bits(d);
    if (e == 0) {
      *reinterpret_cast<uint32_t*>(blk) = static_cast<uint32_t>(dh) | (static_cast<uint32_t>(float_to_f16_bits(sum)) << 16);
    }
    const float dq = f16_bits_to_float(dh);
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = v[i] - dq * static_cast<float>(q[i]);
  }
}

constexpr float kFp16Max = 65504.0f;

// One lane's share (4 of 32 values) of a DS4 group: ties-to-even, clamp +-127, fp16 scale and sum.
__device__ __forceinline__ void ds4_pack_group(const float (&v)[4], float amax, int64_t g, int e, uint8_t* out) {
  const int64_t blk_idx = g >> 2;
  const int grp = static_cast<int>(g & 3);
  const float sum = fminf(kFp16Max, fmaxf(-kFp16Max, oct_tree_sum32(v[0], v[1], v[2], v[3])));
  const float scale = fminf(kFp16Max, amax / 127.0f);
  uint32_t packed = 0;
  if (scale > 0.0f) {
    packed = pack_i8x4(static_cast<int>(fminf(127.0f, fmaxf(-127.0f, rintf(v[0] / scale)))),
                       static_cast<int>(fminf(127.0f, fmaxf(-127.0f, rintf(v[1] / scale)))),
                       static_cast<int>(fminf(127.0f, fmaxf(-127.0f, rintf(v[2] / scale)))),
                       static_cast<int>(fminf(127.0f, fmaxf(-127.0f, rintf(v[3] / scale)))));
  }
  uint8_t* blk = out + blk_idx * DS4_BYTES;
  *reinterpret_cast<uint32_t*>(blk + 16 + grp * 32 + 4 * e) = packed;
  if (e == 0) {
    *reinterpret_cast<uint32_t*>(blk + 4 * grp) =
        static_cast<uint32_t>(float_to_f16_bits(scale)) | (static_cast<uint32_t>(float_to_f16_bits(sum)) << 16);
  }
}

// One lane's share (4 of 32 values) of a D4S4 group: ties away from zero, clamp -128..127, float32 scale and sum
// (four sequential adds per lane, then an xor tree over the 8 lanes: 4, 2, 1).
__device__ __forceinline__ void d4s4_pack_group(const float (&v)[4], float amax, int64_t g, int e, uint8_t* out) {
  const int64_t blk_idx = g >> 2;
  const int grp = static_cast<int>(g & 3);
  float s = ((v[0] + v[1]) + v[2]) + v[3];
  s += dpp_f<DPP_ROW_SHL4>(s);
  s += dpp_f<DPP_ROW_SHL2>(s);
  s += dpp_f<DPP_ROW_SHL1>(s);
  const float d = amax == 0.0f ? 0.0f : amax / 127.0f;
  uint32_t packed = 0;
  if (d != 0.0f) {
    packed = pack_i8x4(max(-128, min(127, static_cast<int>(roundf(v[0] / d)))),
                       max(-128, min(127, static_cast<int>(roundf(v[1] / d)))),
                       max(-128, min(127, static_cast<int>(roundf(v[2] / d)))),
                       max(-128, min(127, static_cast<int>(roundf(v[3] / d)))));
  }
  uint8_t* blk = out + blk_idx * D4S4_BYTES;
  *reinterpret_cast<uint32_t*>(blk + 32 + grp * 32 + 4 * e) = packed;
  if (e == 0) {
    *reinterpret_cast<float*>(blk + 4 * grp) = d;
    *reinterpret_cast<float*>(blk + 16 + 4 * grp) = s;
  }
}

// DS4 (ties-to-even, clamp +-127, fp16 scale and sum) or D4S4 (ties away,
// clamp -128..127, float32 scale and sum).  One group of 8 lanes per 32 values;
// a 128-value block is four consecutive groups.
template <bool D4S4>
__global__ void __launch_bounds__(256) pack_mmq_kernel(const uint16_t* __restrict__ x, uint8_t* __restrict__ out,
                                                       int64_t total_groups) {
  const int64_t g = static_cast<int64_t>(blockIdx.x) * 32 + (threadIdx.x >> 3);
  const int e = threadIdx.x & 7;
  if (g >= total_groups) return;
  float v[4];
  load4_values(x, KIND_BF16, g * 32 + e * 4, v);
  const float amax = oct_max(fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3]))));
  if constexpr (D4S4) {
    d4s4_pack_group(v, amax, g, e, out);
  } else {
    ds4_pack_group(v, amax, g, e, out);
  }
}

// gate_up [rows, 2*inter] (gate columns first) -> DS4 blocks of bf16_round(silu(gate) * up):
// the bytes the two-step path (SiLU*up to bf16, then the DS4 pack) produces.
template <bool D4S4>
__global__ void __launch_bounds__(256) silu_mul_ds4_pack_kernel(const void* __restrict__ gate_up, int in_kind,
                                                                uint8_t* __restrict__ out, int64_t total_groups,
                                                                int64_t inter) {
  const int64_t g = static_cast<int64_t>(blockIdx.x) * 32 + (threadIdx.x >> 3);
  const int e = threadIdx.x & 7;
  if (g >= total_groups) return;
  const int64_t flat = g * 32 + e * 4;
  const int64_t row = flat / inter, col = flat - row * inter;
  float gate[4], up[4], v[4];
  load4_values(gate_up, in_kind, row * 2 * inter + col, gate);
  load4_values(gate_up, in_kind, row * 2 * inter + inter + col, up);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float sig = 1.0f / (1.0f + expf(-gate[i]));
    v[i] = bf16_bits_to_float(float_to_bf16_bits(gate[i] * sig * up[i]));
  }
  const float amax = oct_max(fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3]))));
  if constexpr (D4S4) {
    d4s4_pack_group(v, amax, g, e, out);
  } else {
    ds4_pack_group(v, amax, g, e, out);
  }
}

// The DS4 pack of rows gathered through the routing index: output row r is the pack of token
// sorted_lanes[r] / top_k; a negative lane or a token outside [0, tokens) packs as a row of zeros
// (gguf_q4_k_q8_1_selected_prefill.hip:705-772).  Bytes equal a row gather followed by the plain pack.
__global__ void __launch_bounds__(256) gather_ds4_pack_kernel(const uint16_t* __restrict__ hidden_states,
                                                              const int64_t* __restrict__ sorted_lanes,
                                                              uint8_t* __restrict__ out, int64_t total_groups,
                                                              int64_t groups_per_row, int64_t tokens, int64_t top_k) {
  const int64_t g = static_cast<int64_t>(blockIdx.x) * 32 + (threadIdx.x >> 3);
  const int e = threadIdx.x & 7;
  if (g >= total_groups) return;
  const int64_t row = g / groups_per_row, within = g - row * groups_per_row;
  const int64_t lane = sorted_lanes[row];
  const int64_t token = lane >= 0 ? lane / top_k : -1;
  float v[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  if (token >= 0 && token < tokens) load4_values(hidden_states, KIND_BF16, (token * groups_per_row + within) * 32 + e * 4, v);
  const float amax = oct_max(fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3]))));
  ds4_pack_group(v, amax, g, e, out);
}

int launch_q8_1(const void* x, int kind, void* xq, int64_t rows, int64_t in_features, hipStream_t stream) {
  if (!x || !xq || rows <= 0 || in_features <= 0 || (in_features % 32) != 0) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  const int64_t groups = rows * (in_features / 32);
  const int64_t grid = (groups + 31) / 32;
  if (grid > 0x7FFFFFFF) return static_cast<int>(hipErrorInvalidValue);
  hipLaunchKernelGGL(quantize_q8_1_kernel, dim3(static_cast<unsigned>(grid)), dim3(256), 0, stream, x, kind,
                     static_cast<uint8_t*>(xq), groups);
  return static_cast<int>(hipGetLastError());
}

template <bool D4S4>
int launch_pack(const void* x, void* out, int64_t rows, int64_t hidden, hipStream_t stream) {
  if (!x || !out || rows <= 0 || hidden <= 0 || (hidden % 128) != 0) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  const int64_t groups = rows * (hidden / 32);
  const int64_t grid = (groups + 31) / 32;
  if (grid > 0x7FFFFFFF) return static_cast<int>(hipErrorInvalidValue);
  hipLaunchKernelGGL(pack_mmq_kernel<D4S4>, dim3(static_cast<unsigned>(grid)), dim3(256), 0, stream,
                     static_cast<const uint16_t*>(x), static_cast<uint8_t*>(out), groups);
  return static_cast<int>(hipGetLastError());
}

}  // namespace

extern "C" int hipengine_gguf_q4_k_quantize_f32_q8_1(const void* x, void* xq, int64_t rows, int64_t in_features,
                                                     hipStream_t stream) {
  return launch_q8_1(x, KIND_F32, xq, rows, in_features, stream);
}

extern "C" int hipengine_gguf_q4_k_quantize_bf16_q8_1(const void* x, void* xq, int64_t rows, int64_t in_features,
                                                      hipStream_t stream) {
  return launch_q8_1(x, KIND_BF16, xq, rows, in_features, stream);
}

extern "C" int hipengine_gguf_q4_k_quantize_bf16_q8_1x2(const void* x, void* xq, int64_t rows, int64_t in_features,
                                                        hipStream_t stream) {
  if (!x || !xq || rows <= 0 || in_features <= 0 || (in_features % 32) != 0) return static_cast<int>(hipErrorInvalidValue);
  const int64_t groups = rows * (in_features / 32);
  const int64_t grid = (groups + 31) / 32;
  if (grid > 0x7FFFFFFF) return static_cast<int>(hipErrorInvalidValue);
  hipLaunchKernelGGL(quantize_q8_1x2_kernel, dim3(static_cast<unsigned>(grid)), dim3(256), 0, stream, x, KIND_BF16,
                     static_cast<uint8_t*>(xq), groups);
  return static_cast<int>(hipGetLastError());
}

extern "C" int hipengine_gguf_q8_1_mmq_ds4_pack_bf16(const void* x, void* out, int64_t rows, int64_t hidden,
                                                     hipStream_t stream) {
  return launch_pack<false>(x, out, rows, hidden, stream);
}

extern "C" int hipengine_gguf_q8_1_mmq_gather_ds4_pack_bf16(const uint16_t* hidden_states, const int64_t* sorted_lanes,
                                                            void* out, int64_t rows, int64_t hidden, int64_t tokens,
                                                            int64_t top_k, hipStream_t stream) {
  if (!hidden_states || !sorted_lanes || !out || rows <= 0 || hidden <= 0 || (hidden % 128) != 0 || tokens <= 0 ||
      top_k <= 0) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  const int64_t groups = rows * (hidden / 32);
  const int64_t grid = (groups + 31) / 32;
  if (grid > 0x7FFFFFFF) return static_cast<int>(hipErrorInvalidValue);
  hipLaunchKernelGGL(gather_ds4_pack_kernel, dim3(static_cast<unsigned>(grid)), dim3(256), 0, stream, hidden_states,
                     sorted_lanes, static_cast<uint8_t*>(out), groups, hidden / 32, tokens, top_k);
  return static_cast<int>(hipGetLastError());
}

extern "C" int hipengine_gguf_q8_1_d4s4_f32_quantize_bf16(const void* x, void* out, int64_t rows, int64_t hidden,
                                                          hipStream_t stream) {
  return launch_pack<true>(x, out, rows, hidden, stream);
}

extern "C" int hipengine_gfx950_moe_silu_mul_ds4_pack(const void* gate_up, int in_kind, void* out, int64_t rows,
                                                      int64_t inter, hipStream_t stream) {
  if (!gate_up || !out || rows <= 0 || inter <= 0 || (inter % 128) != 0 || in_kind < KIND_F32 || in_kind > KIND_F16) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  const int64_t groups = rows * (inter / 32);
  const int64_t grid = (groups + 31) / 32;
  if (grid > 0x7FFFFFFF) return static_cast<int>(hipErrorInvalidValue);
  hipLaunchKernelGGL(silu_mul_ds4_pack_kernel<false>, dim3(static_cast<unsigned>(grid)), dim3(256), 0, stream, gate_up,
                     in_kind, static_cast<uint8_t*>(out), groups, inter);
  return static_cast<int>(hipGetLastError());
}

// The same into D4S4 blocks (what the Q5_K / Q6_K MMQ kernels take).
extern "C" int hipengine_gfx950_moe_silu_mul_d4s4_pack(const void* gate_up, int in_kind, void* out, int64_t rows,
                                                       int64_t inter, hipStream_t stream) {
  if (!gate_up || !out || rows <= 0 || inter <= 0 || (inter % 128) != 0 || in_kind < KIND_F32 || in_kind > KIND_F16) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  const int64_t groups = rows * (inter / 32);
  const int64_t grid = (groups + 31) / 32;
  if (grid > 0x7FFFFFFF) return static_cast<int>(hipErrorInvalidValue);
  hipLaunchKernelGGL(silu_mul_ds4_pack_kernel<true>, dim3(static_cast<unsigned>(grid)), dim3(256), 0, stream, gate_up,
                     in_kind, static_cast<uint8_t*>(out), groups, inter);
  return static_cast<int>(hipGetLastError());
}

int hipengine_gfx950::quantize_load() {
  hipFuncAttributes attr;
  return static_cast<int>(hipFuncGetAttributes(&attr, reinterpret_cast<const void*>(pack_mmq_kernel<false>)));
}
