// Expert-indexed (MoE) forms of the GGUF k-quant matmul for gfx950, and the
// routing index they consume.
//
//   routing index  selected[L] (lane = token*top_k + slot) -> expert-major order:
//                  expert_start[E+1], sorted_lanes, compact_to_source, sorted_weights,
//                  active list; tile map of 32-row tiles per expert
//                  (kernels/hip_gfx1100/moe/group_scatter.hip:62-141,328-389)
//   decode         selected GEMV: out[lane] = W[selected[lane]] . x[lane / top_k]
//                  (kernels/hip_gfx1100/quant/gguf_q4_k_gemv.hip:322-359), the fused
//                  gate/up form silu(gate)*up (:666-737) and the routed down
//                  projection summed over a token's experts; all on the q8_1
//                  integer GEMV body of gguf_gemv.hpp
//   prefill        expert-grouped Q4_K x DS4 MMQ over compact rows and the tile map
//                  (kernels/hip_gfx1100/quant/gguf_q4_k_q8_1_selected_prefill.hip:1256-1670)
//                  on the tile engine of gguf_mmq_q4k.hpp

#include "gguf_gemv.hpp"
#include "gguf_mmq_q4k.hpp"
#include "gguf_mmq_q6k.hpp"
#include "gguf_mmq_q8_0.hpp"

#include "gguf_init.hpp"

#include "../../include/hipengine_gfx950.h"

namespace {

using namespace hipengine_gfx950;

constexpr int MAX_EXPERTS = 2048;

// --------------------------------------------------------------------------
// routing index
// --------------------------------------------------------------------------

// Exclusive prefix of the per-expert counts in cnt[0..num_experts) (LDS, replaced by the prefix) -> expert_start[0..E],
// and the ascending list of the experts with a non-zero count; all 1024 threads of the workgroup call it after a
// barrier that made cnt complete.  PER consecutive experts per thread, a shuffle scan per wave, the wave totals
// through LDS (a single thread walking 256 counters in LDS costs ~10 us of read latency).
__device__ __forceinline__ void moe_prefix_active_block(int* cnt, int* act, int* totals, int num_experts,
                                                        int64_t* __restrict__ expert_start,
                                                        int64_t* __restrict__ active_experts,
                                                        int64_t* __restrict__ active_count) {
  constexpr int PER = MAX_EXPERTS / 1024;
  __shared__ int wsum[16], wnz[16];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  int c[PER], sum = 0, nz = 0;
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    const int e = tid * PER + k;
    c[k] = e < num_experts ? cnt[e] : 0;
    sum += c[k];
    nz += c[k] > 0 ? 1 : 0;
  }
  int isum = sum, inz = nz;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const int t = __shfl_up(isum, off), u = __shfl_up(inz, off);
    if (lane >= off) { isum += t; inz += u; }
  }
  if (lane == 63) { wsum[wave] = isum; wnz[wave] = inz; }
  __syncthreads();
  int base = 0, base_nz = 0;
  for (int w = 0; w < wave; ++w) { base += wsum[w]; base_nz += wnz[w]; }
  int offset = base + isum - sum, rank = base_nz + inz - nz;
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    const int e = tid * PER + k;
    if (e < num_experts) {
      cnt[e] = offset;
      if (c[k] > 0) act[rank++] = e;
      offset += c[k];
    }
  }
  if (tid == 1023) { totals[0] = base + isum; totals[1] = base_nz + inz; }
  __syncthreads();
  for (int e = threadIdx.x; e < num_experts; e += 1024) expert_start[e] = cnt[e];
  if (active_experts)
    for (int i = threadIdx.x; i < totals[1]; i += 1024) active_experts[i] = act[i];
  if (threadIdx.x == 0) {
    expert_start[num_experts] = totals[0];
    if (active_count) active_count[0] = totals[1];
  }
}

// One workgroup: histogram of the selected experts in LDS (integer atomics, so the
// result does not depend on order), exclusive prefix -> expert_start[0..E],
// ascending list of the experts that own at least one lane.
template <class ID>
__global__ void __launch_bounds__(1024) moe_count_prefix_kernel(const ID* __restrict__ selected,
                                                                int64_t* __restrict__ expert_start,
                                                                int64_t* __restrict__ active_experts,
                                                                int64_t* __restrict__ active_count,
                                                                int64_t* __restrict__ lane_to_compact, int64_t lanes,
                                                                int num_experts) {
  __shared__ int cnt[MAX_EXPERTS];
  __shared__ int act[MAX_EXPERTS];
  __shared__ int totals[2];
  for (int e = threadIdx.x; e < num_experts; e += 1024) cnt[e] = 0;
  __syncthreads();
  // eight loads in flight per thread: the loop is otherwise a chain of global-memory round trips
  for (int64_t i0 = threadIdx.x; i0 < lanes; i0 += 8 * 1024) {
    int64_t e[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int64_t i = i0 + u * 1024;
      e[u] = i < lanes ? selected[i] : -1;
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      if (e[u] >= 0 && e[u] < num_experts) atomicAdd(&cnt[static_cast<int>(e[u])], 1);
      else if (lane_to_compact && i0 + u * 1024 < lanes) lane_to_compact[i0 + u * 1024] = -1;   // a lane of no expert
    }
  }
  __syncthreads();
  moe_prefix_active_block(cnt, act, totals, num_experts, expert_start, active_experts, active_count);
}

// The prefix and the active list from counts that are already in memory (one workgroup of 1024 threads).
__global__ void __launch_bounds__(1024) moe_prefix_active_kernel(const int32_t* __restrict__ counts,
                                                                 int64_t* __restrict__ expert_start,
                                                                 int64_t* __restrict__ active_experts,
                                                                 int64_t* __restrict__ active_count, int num_experts) {
  __shared__ int cnt[MAX_EXPERTS];
  __shared__ int act[MAX_EXPERTS];
  __shared__ int totals[2];
  for (int e = threadIdx.x; e < num_experts; e += 1024) cnt[e] = counts[e] > 0 ? counts[e] : 0;
  __syncthreads();
  moe_prefix_active_block(cnt, act, totals, num_experts, expert_start, active_experts, active_count);
}

// One workgroup per expert: writes its lanes in ascending lane order (wave
// ballots keep the order) into [expert_start[e], expert_start[e+1]).
template <class ID>
__global__ void __launch_bounds__(1024) moe_place_kernel(const ID* __restrict__ selected,
                                                         const float* __restrict__ routing,
                                                         const int64_t* __restrict__ expert_start,
                                                         int64_t* __restrict__ sorted_lanes,
                                                         int64_t* __restrict__ sorted_experts,
                                                         int64_t* __restrict__ compact_to_source,
                                                         float* __restrict__ sorted_weights,
                                                         int64_t* __restrict__ lane_to_compact, int64_t lanes,
                                                         int64_t top_k) {
  __shared__ int wave_cnt[2][16];
  const int64_t e = blockIdx.x;
  const int64_t base = expert_start[e];
  const int count = static_cast<int>(expert_start[e + 1] - base);
  if (count <= 0) return;
  const int lane_id = threadIdx.x & 63, wave = threadIdx.x >> 6;
  constexpr int PER = 4;                        // consecutive lanes per thread and chunk
  constexpr int64_t CHUNK = 1024 * PER;
  int running = 0, buf = 0;
  // the selections of the next chunk are loaded before this chunk's barrier
  int64_t sel_next[PER];
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const int64_t lane = static_cast<int64_t>(threadIdx.x) * PER + j;
    sel_next[j] = lane < lanes ? selected[lane] : -1;
  }
  for (int64_t chunk = 0; chunk < lanes && running < count; chunk += CHUNK, buf ^= 1) {
    const int64_t lane0 = chunk + static_cast<int64_t>(threadIdx.x) * PER;
    bool flag[PER];
    int mine = 0;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      flag[j] = lane0 + j < lanes && sel_next[j] == e;
      mine += flag[j] ? 1 : 0;
      sel_next[j] = lane0 + CHUNK + j < lanes ? selected[lane0 + CHUNK + j] : -1;
    }
    // lanes of this expert in the threads before this one of the wave (ascending lane order: thread, then j)
    int before = 0, wave_total = 0;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const unsigned long long ballot = __ballot(flag[j]);
      before += __popcll(ballot & ((1ull << lane_id) - 1ull));
      wave_total += __popcll(ballot);
    }
    if (lane_id == 0) wave_cnt[buf][wave] = wave_total;
    __syncthreads();      // one barrier per chunk: the count buffers alternate
    int offset = running, total = 0;
#pragma unroll
    for (int w = 0; w < 16; ++w) {
      const int c = wave_cnt[buf][w];
      if (w < wave) offset += c;
      total += c;
    }
    if (mine) {
      int64_t idx = base + offset + before;
#pragma unroll
      for (int j = 0; j < PER; ++j) {
        if (flag[j]) {
          const int64_t lane = lane0 + j;
          sorted_lanes[idx] = lane;
          if (sorted_experts) sorted_experts[idx] = e;
          if (compact_to_source) compact_to_source[idx] = lane / top_k;
          if (sorted_weights) sorted_weights[idx] = routing[lane];
          if (lane_to_compact) lane_to_compact[lane] = idx;
          ++idx;
        }
      }
    }
    running += total;
  }
}

template <class ID>
int launch_compact(const ID* selected, const float* routing, int64_t* expert_start, int64_t* active_experts,
                   int64_t* active_count, int64_t* sorted_lanes, int64_t* sorted_experts, int64_t* compact_to_source,
                   float* sorted_weights, int64_t lanes, int64_t num_experts, int64_t top_k, hipStream_t stream,
                   int64_t* lane_to_compact = nullptr) {
  if (!selected || !expert_start || !sorted_lanes || (sorted_weights && !routing) || lanes <= 0 || lanes > (1ll << 30) ||
      num_experts <= 0 || num_experts > MAX_EXPERTS || top_k <= 0) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  hipLaunchKernelGGL(moe_count_prefix_kernel<ID>, dim3(1), dim3(1024), 0, stream, selected, expert_start, active_experts,
                     active_count, lane_to_compact, lanes, static_cast<int>(num_experts));
  hipLaunchKernelGGL(moe_place_kernel<ID>, dim3(static_cast<unsigned>(num_experts)), dim3(1024), 0, stream, selected, routing,
                     expert_start, sorted_lanes, sorted_experts, compact_to_source, sorted_weights, lane_to_compact, lanes,
                     top_k);
  return static_cast<int>(hipGetLastError());
}

// One workgroup: per-expert row counts rounded up to tile_rows, their prefix,
// and the tile -> expert map (-1 where a tile belongs to no expert).
__global__ void __launch_bounds__(256) moe_tile_map_kernel(const int64_t* __restrict__ expert_start_compact,
                                                           int64_t* __restrict__ tile_expert_start,
                                                           int64_t* __restrict__ tile_expert,
                                                           int64_t* __restrict__ total_out, int num_experts,
                                                           int64_t tile_capacity, int tile_rows) {
  __shared__ int start[MAX_EXPERTS + 1];
  for (int e = threadIdx.x; e < num_experts; e += 256) {
    const int c = static_cast<int>(expert_start_compact[e + 1] - expert_start_compact[e]);
    start[e] = (c + tile_rows - 1) / tile_rows * tile_rows;
  }
  for (int64_t i = threadIdx.x; i < tile_capacity; i += 256) tile_expert[i] = -1;
  __syncthreads();
  {
    constexpr int PER = MAX_EXPERTS / 256;   // consecutive experts per thread
    __shared__ int wsum[4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int c[PER], sum = 0;
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      const int e = tid * PER + k;
      c[k] = e < num_experts ? start[e] : 0;
      sum += c[k];
    }
    int isum = sum;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const int t = __shfl_up(isum, off);
      if (lane >= off) isum += t;
    }
    if (lane == 63) wsum[wave] = isum;
    __syncthreads();
    int base = 0;
    for (int w = 0; w < wave; ++w) base += wsum[w];
    int offset = base + isum - sum;
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      const int e = tid * PER + k;
      if (e < num_experts) { start[e] = offset; offset += c[k]; }
    }
    if (tid == 255) start[num_experts] = base + isum;
  }
  __syncthreads();
  for (int e = threadIdx.x; e <= num_experts; e += 256) tile_expert_start[e] = start[e];
  if (threadIdx.x == 0) total_out[0] = start[num_experts];
  for (int e = threadIdx.x; e < num_experts; e += 256) {
    for (int t = start[e] / tile_rows; t < start[e + 1] / tile_rows; ++t)
      if (tile_capacity <= 0 || t < tile_capacity) tile_expert[t] = e;
  }
}

int launch_tile_map(const int64_t* expert_start_compact, int64_t* tile_expert_start, int64_t* tile_expert,
                    int64_t* total_out, int64_t num_experts, int64_t tile_capacity, int tile_rows,
                    hipStream_t stream) {
  if (!expert_start_compact || !tile_expert_start || !tile_expert || !total_out || num_experts <= 0 ||
      num_experts > MAX_EXPERTS || tile_rows <= 0) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  hipLaunchKernelGGL(moe_tile_map_kernel, dim3(1), dim3(256), 0, stream, expert_start_compact, tile_expert_start,
                     tile_expert, total_out, static_cast<int>(num_experts), tile_capacity, tile_rows);
  return static_cast<int>(hipGetLastError());
}

// lane_to_compact[lane] = position of the lane in the expert-major order, -1 if dropped.
__global__ void moe_fill_i64_kernel(int64_t* p, int64_t n, int64_t v) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) p[i] = v;
}
__global__ void moe_invert_kernel(const int64_t* __restrict__ sorted_lanes, int64_t* __restrict__ lane_to_compact,
                                  int64_t compact_rows, int64_t lanes) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < compact_rows) {
    const int64_t lane = sorted_lanes[i];
    if (lane >= 0 && lane < lanes) lane_to_compact[lane] = i;
  }
}

// ---- the count / prefix / scatter pipeline hipEngine's runner drives step by step ----
// (runtime/qwen35_gguf_runner.py:34107-34143; kernels moe/group_scatter.hip:9-60,391-485)

// counts[e] += lanes routed to e.  The caller zeroes counts (int32), as in hipEngine.
__global__ void __launch_bounds__(256) moe_group_count_kernel(const int64_t* __restrict__ selected,
                                                              int32_t* __restrict__ counts, int64_t lanes,
                                                              int64_t num_experts) {
  const int64_t lane = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (lane >= lanes) return;
  const int64_t e = selected[lane];
  if (e >= 0 && e < num_experts) atomicAdd(&counts[e], 1);
}

// One workgroup of 1024: padded_counts[e] = counts[e] rounded up to pad_multiple, expert_start = its
// exclusive prefix, expert_start[E] = total_padded[0] = the sum.
__global__ void __launch_bounds__(1024) moe_group_prefix_kernel(const int32_t* __restrict__ counts,
                                                                int32_t* __restrict__ padded_counts,
                                                                int64_t* __restrict__ expert_start,
                                                                int64_t* __restrict__ total_padded, int num_experts,
                                                                int64_t pad_multiple) {
  constexpr int PER = MAX_EXPERTS / 1024;
  __shared__ int64_t wsum[16];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  int64_t c[PER], sum = 0;
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    const int e = tid * PER + k;
    int64_t padded = 0;
    if (e < num_experts) {
      const int64_t n = counts[e];
      padded = pad_multiple > 1 ? (n + pad_multiple - 1) / pad_multiple * pad_multiple : n;
      padded_counts[e] = static_cast<int32_t>(padded);
    }
    c[k] = padded;
    sum += padded;
  }
  int64_t isum = sum;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const int64_t t = __shfl_up(isum, off);
    if (lane >= off) isum += t;
  }
  if (lane == 63) wsum[wave] = isum;
  __syncthreads();
  int64_t base = 0;
  for (int w = 0; w < wave; ++w) base += wsum[w];
  int64_t offset = base + isum - sum;
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    const int e = tid * PER + k;
    if (e < num_experts) { expert_start[e] = offset; offset += c[k]; }
  }
  if (tid == 1023) {
    expert_start[num_experts] = base + isum;
    total_padded[0] = base + isum;
  }
}

// One workgroup per expert: the expert's lanes in ascending lane order from expert_start[e] on (hipEngine's
// scatter takes its slots with atomics, in whatever order the lanes arrive; ascending order is one of the
// orders it can produce), scatter_offsets[e] += the number placed, as the atomics would leave it.
__global__ void __launch_bounds__(1024) moe_scatter_kernel(const int64_t* __restrict__ selected,
                                                           const float* __restrict__ routing,
                                                           const int64_t* __restrict__ expert_start,
                                                           int32_t* __restrict__ scatter_offsets,
                                                           int64_t* __restrict__ sorted_lanes,
                                                           int64_t* __restrict__ sorted_experts,
                                                           float* __restrict__ sorted_weights, int64_t lanes,
                                                           const uint16_t* __restrict__ hidden,
                                                           uint16_t* __restrict__ packed, int64_t top_k,
                                                           int64_t hidden_size) {
  __shared__ int wave_cnt[2][16];
  const int64_t e = blockIdx.x;
  const int64_t base = expert_start[e] + scatter_offsets[e];
  const int lane_id = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int running = 0, buf = 0;
  for (int64_t chunk = 0; chunk < lanes; chunk += 1024, buf ^= 1) {
    const int64_t lane = chunk + threadIdx.x;
    const bool flag = lane < lanes && selected[lane] == e;
    const unsigned long long ballot = __ballot(flag);
    const int before = __popcll(ballot & ((1ull << lane_id) - 1ull));
    if (lane_id == 0) wave_cnt[buf][wave] = __popcll(ballot);
    __syncthreads();
    int offset = running, total = 0;
#pragma unroll
    for (int w = 0; w < 16; ++w) {
      const int c = wave_cnt[buf][w];
      if (w < wave) offset += c;
      total += c;
    }
    if (flag) {
      const int64_t idx = base + offset + before;
      sorted_lanes[idx] = lane;
      if (sorted_experts) sorted_experts[idx] = e;
      if (sorted_weights) sorted_weights[idx] = routing[lane];
    }
    running += total;
  }
  __syncthreads();   // the lanes this workgroup placed are visible to all of its threads
  if (threadIdx.x == 0) scatter_offsets[e] += running;
  // gather: packed[base + i, :] = hidden[sorted_lanes[base + i] / top_k, :] for the rows placed above
  if (hidden && packed) {
    const bool wide = (hidden_size & 7) == 0 &&
                      ((reinterpret_cast<uintptr_t>(hidden) | reinterpret_cast<uintptr_t>(packed)) & 15u) == 0;
    const int64_t per_row = wide ? hidden_size / 8 : hidden_size;
    for (int64_t i = threadIdx.x; i < running * per_row; i += 1024) {
      const int64_t r = i / per_row, c = i - r * per_row;
      const int64_t token = sorted_lanes[base + r] / top_k;
      if (wide) {
        reinterpret_cast<uint4*>(packed + (base + r) * hidden_size)[c] =
            reinterpret_cast<const uint4*>(hidden + token * hidden_size)[c];
      } else {
        packed[(base + r) * hidden_size + c] = hidden[token * hidden_size + c];
      }
    }
  }
}

// packed[row, :] = hidden[sorted_lanes[row] / top_k, :] (16-bit elements), zeros for a negative lane or a
// token outside [0, tokens).  16 bytes per thread where the row length allows.
__global__ void __launch_bounds__(256) moe_gather_rows_kernel(const uint16_t* __restrict__ hidden,
                                                              const int64_t* __restrict__ sorted_lanes,
                                                              uint16_t* __restrict__ packed, int64_t rows,
                                                              int64_t tokens, int64_t top_k, int64_t hidden_size) {
  const int64_t row = blockIdx.x;
  if (row >= rows) return;
  const int64_t lane = sorted_lanes[row];
  const int64_t token = lane >= 0 ? lane / top_k : -1;
  const bool valid = token >= 0 && token < tokens;
  const uint16_t* src = hidden + (valid ? token : 0) * hidden_size;
  uint16_t* dst = packed + row * hidden_size;
  if ((hidden_size & 7) == 0 && ((reinterpret_cast<uintptr_t>(hidden) | reinterpret_cast<uintptr_t>(packed)) & 15u) == 0) {
    for (int64_t c = threadIdx.x; c < hidden_size / 8; c += blockDim.x) {
      uint4 v = make_uint4(0u, 0u, 0u, 0u);
      if (valid) v = reinterpret_cast<const uint4*>(src)[c];
      reinterpret_cast<uint4*>(dst)[c] = v;
    }
  } else {
    for (int64_t c = threadIdx.x; c < hidden_size; c += blockDim.x) dst[c] = valid ? src[c] : static_cast<uint16_t>(0);
  }
}

// --------------------------------------------------------------------------
// elementwise steps between the projections
// --------------------------------------------------------------------------

__device__ __forceinline__ float silu_mul(float gate, float up) {
  const float sig = 1.0f / (1.0f + expf(-gate));
  return gate * sig * up;
}

// gate_up [rows, 2*inter] (gate columns first) -> out [rows, inter] = silu(gate) * up
__global__ void moe_silu_mul_kernel(const void* __restrict__ gate_up, void* __restrict__ out, int64_t rows,
                                    int64_t inter, int in_kind, int out_kind) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= rows * inter) return;
  const int64_t r = i / inter, c = i - r * inter;
  const float g = load_scalar(gate_up, r * 2 * inter + c, in_kind);
  const float u = load_scalar(gate_up, r * 2 * inter + inter + c, in_kind);
  store_scalar(out, i, silu_mul(g, u), out_kind);
}

// out[t, h] = sum over the token's slots, in slot order, of routing[lane] * down[lane_to_compact[lane], h]
__global__ void moe_weighted_gather_kernel(const void* __restrict__ down, const int64_t* __restrict__ lane_to_compact,
                                           const float* __restrict__ routing, void* __restrict__ out, int64_t tokens,
                                           int64_t top_k, int64_t hidden, int64_t compact_rows, int in_kind,
                                           int out_kind) {
  const int64_t t = blockIdx.y;
  const int64_t h = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (t >= tokens || h >= hidden) return;
  float acc = 0.0f;
  for (int64_t s = 0; s < top_k; ++s) {
    const int64_t lane = t * top_k + s;
    const int64_t c = lane_to_compact[lane];
    if (c < 0 || c >= compact_rows) continue;
    acc += routing[lane] * load_scalar(down, c * hidden + h, in_kind);
  }
  store_scalar(out, t * hidden + h, acc, out_kind);
}

// The same sums for hidden % 8 == 0 and top_k <= 8, eight consecutive features per thread: a token's slot
// indices and weights are fetched first, then all of its rows' 16- or 32-byte pieces are in flight together
// (the scalar form above is a chain of top_k dependent 2- or 4-byte loads per thread).
template <int IN_KIND>
__global__ void __launch_bounds__(256) moe_weighted_gather8_kernel(const void* __restrict__ down,
                                                                   const int64_t* __restrict__ lane_to_compact,
                                                                   const float* __restrict__ routing,
                                                                   void* __restrict__ out, int64_t tokens, int top_k,
                                                                   int64_t hidden, int64_t compact_rows, int out_kind) {
  const int64_t t = blockIdx.y;
  const int64_t h = (static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x) * 8;
  if (t >= tokens || h >= hidden) return;
  int64_t c[8];
  float wgt[8];
#pragma unroll
  for (int s = 0; s < 8; ++s) {
    const bool on = s < top_k;
    c[s] = on ? lane_to_compact[t * top_k + s] : -1;
    wgt[s] = on ? routing[t * top_k + s] : 0.0f;
  }
  float v[8][8];
#pragma unroll
  for (int s = 0; s < 8; ++s) {
    const bool live = c[s] >= 0 && c[s] < compact_rows;
    const int64_t base = (live ? c[s] : 0) * hidden + h;
    if constexpr (IN_KIND == KIND_F32) {
      const float4 lo = *reinterpret_cast<const float4*>(static_cast<const float*>(down) + base);
      const float4 hi = *reinterpret_cast<const float4*>(static_cast<const float*>(down) + base + 4);
      v[s][0] = lo.x; v[s][1] = lo.y; v[s][2] = lo.z; v[s][3] = lo.w;
      v[s][4] = hi.x; v[s][5] = hi.y; v[s][6] = hi.z; v[s][7] = hi.w;
    } else {
      const uint4 p = *reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(down) + base);
      const uint32_t w32[4] = {p.x, p.y, p.z, p.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        v[s][2 * e] = IN_KIND == KIND_BF16 ? bf16_bits_to_float(w32[e] & 0xFFFFu) : f16_bits_to_float(w32[e] & 0xFFFFu);
        v[s][2 * e + 1] = IN_KIND == KIND_BF16 ? bf16_bits_to_float(w32[e] >> 16) : f16_bits_to_float(w32[e] >> 16);
      }
    }
  }
  float res[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    float acc = 0.0f;
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      if (s < top_k && c[s] >= 0 && c[s] < compact_rows) acc += wgt[s] * v[s][e];
    }
    res[e] = acc;
  }
  if (out_kind == KIND_F32) {
    float* o = static_cast<float*>(out) + t * hidden + h;
    *reinterpret_cast<float4*>(o) = float4{res[0], res[1], res[2], res[3]};
    *reinterpret_cast<float4*>(o + 4) = float4{res[4], res[5], res[6], res[7]};
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) store_scalar(out, t * hidden + h + e, res[e], out_kind);
  }
}

// --------------------------------------------------------------------------
// decode: selected GEMV on the q8_1 integer GEMV body
// --------------------------------------------------------------------------

enum SelMode : int { SEL_SINGLE = 0, SEL_DUAL_SILU = 1, SEL_DOWN_SUM = 2, SEL_DUAL = 3 };

struct SelArgs {
  GemvArgs g;                 // x, w (first weight), out, kinds, K, N, ks, nrg; rows = 1
  const uint8_t* w_b;         // second weight (dual)
  void* out_b;                // second output (SEL_DUAL)
  const int64_t* selected;    // [lanes]
  const float* routing;       // [lanes] (down sum)
  int x_rows;                 // activation rows (tokens) for single/dual; tokens for down sum
  int lanes;
  int num_experts;
  int top_k;
  int round_mid;              // dual: round gate and up to the output type before silu (the fused device form)
  int pair_offset;            // dual: byte offset in LDS of the [2][rows] gate/up exchange buffer
};

__device__ __forceinline__ int64_t scalar_bytes(int kind) { return kind == KIND_F32 ? 4 : 2; }
// bytes of one activation row of K values: scalars, or 36-byte q8_1 blocks
__device__ __forceinline__ int64_t act_row_bytes(int kind, int K) {
  return kind == KIND_Q8_1 ? static_cast<int64_t>(K / 32) * Q8_1_BYTES : static_cast<int64_t>(K) * scalar_bytes(kind);
}

// Workgroup size cap: the CB weight blocks of a chunk have to fit the VGPR
// budget the cap implies (128 registers at 1024 threads, 256 at 512).
template <int QT, int BLOCKS>
constexpr int sel_max_threads() {
  return BLOCKS * GemvTraits<QT>::REGS <= 48 ? 1024 : 512;
}

// XK >= 0 fixes the activation kind at compile time (a decode kernel runs its staging code once, with a cold
// instruction cache: the code of the other kinds is launch latency), XK < 0 reads it from the arguments.
template <int QT, int R, int CB, int MODE, int XK = -1>
__global__ void __launch_bounds__((sel_max_threads<QT, R * CB>())) selected_gemv_kernel(SelArgs s) {
  extern __shared__ __align__(16) uint8_t smem[];
  if constexpr (XK >= 0) s.g.x_kind = XK;
  const int64_t row_bytes = static_cast<int64_t>(s.g.K / QK_K) * GemvTraits<QT>::SUPER_BYTES;
  const int64_t expert_bytes = static_cast<int64_t>(s.g.N) * row_bytes;
  GemvArgs a = s.g;
  a.rows = 1;
  const int lane = blockIdx.y;
  const int64_t e = s.selected[lane];
  if (e < 0 || e >= s.num_experts) return;
  const int per = s.lanes / s.x_rows;
  const int x_row = s.x_rows == 1 ? 0 : lane / per;
  a.x = static_cast<const uint8_t*>(s.g.x) + static_cast<int64_t>(x_row) * act_row_bytes(s.g.x_kind, s.g.K);
  if constexpr (XK == KIND_SILU_BF16) {
    a.x_up = static_cast<const uint8_t*>(s.g.x_up) + static_cast<int64_t>(x_row) * act_row_bytes(s.g.x_kind, s.g.K);
  }
  a.out = static_cast<uint8_t*>(s.g.out) + static_cast<int64_t>(lane) * s.g.N * scalar_bytes(s.g.out_kind);
  if constexpr (MODE == SEL_SINGLE) {
    gemv_workgroup<QT, 1, R, CB>(a, s.g.w + e * expert_bytes, blockIdx.x * s.g.nrg * 16 * R, smem);
  } else if constexpr (MODE == SEL_DUAL) {
    // gate and up rows of the same index in one pass, each stored to its own output
    static_assert(R == 2, "the dual form pairs two matrices");
    void* out_b = static_cast<uint8_t*>(s.out_b) + static_cast<int64_t>(lane) * s.g.N * scalar_bytes(s.g.out_kind);
    gemv_workgroup_emit<QT, 1, 2, CB, true>(
        a, s.g.w + e * expert_bytes, blockIdx.x * s.g.nrg * 16, smem,
        [&](int which, int row, float v) { store_scalar(which ? out_b : a.out, row, v, a.out_kind); },
        s.w_b + e * expert_bytes);
  } else {
    // gate and up rows of the same index in one pass: one staging of the activations,
    // all weight loads of both matrices in flight together
    static_assert(R == 2, "the gate/up form pairs two matrices");
    const int rows_out = s.g.nrg * 16;
    const int first_row = blockIdx.x * rows_out;
    float* pair = reinterpret_cast<float*>(smem + s.pair_offset);      // [2][rows_out]
    gemv_workgroup_emit<QT, 1, 2, CB, true>(
        a, s.g.w + e * expert_bytes, first_row, smem,
        [&](int which, int row, float v) { pair[which * rows_out + (row - first_row)] = v; }, s.w_b + e * expert_bytes);
    __syncthreads();
    const int i = threadIdx.x;
    if (i < rows_out && first_row + i < s.g.N) {
      float gv = pair[i], uv = pair[rows_out + i];
      if (s.round_mid && a.out_kind == KIND_BF16) {
        gv = bf16_bits_to_float(float_to_bf16_bits(gv));
        uv = bf16_bits_to_float(float_to_bf16_bits(uv));
      } else if (s.round_mid && a.out_kind == KIND_F16) {
        gv = f16_bits_to_float(float_to_f16_bits(gv));
        uv = f16_bits_to_float(float_to_f16_bits(uv));
      }
      store_scalar(a.out, first_row + i, silu_mul(gv, uv), a.out_kind);
    }
  }
}

// Routed down projection of one token: out[t, row] = sum over slots s, in slot order, of
// routing[t*top_k + s] * (W[selected[t*top_k + s]] . x[t*top_k + s]).
// One workgroup per (16 output rows, token); its waves are (slot, K slice) pairs, so the
// weight blocks of all the token's experts are in flight together and the activations
// of all slots (top_k consecutive rows of x) are quantized in one pass per K chunk.
template <int QT, int TK, int RG, int XK = -1>
__global__ void __launch_bounds__(1024) selected_down_sum_kernel(SelArgs s) {
  extern __shared__ __align__(16) uint8_t smem[];
  if constexpr (XK >= 0) s.g.x_kind = XK;
  using Regs = WeightRegs<GemvTraits<QT>::REGS>;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int ks = s.g.ks;                       // K slices per slot; waves = TK * ks
  const int slot = wave / ks, kslice = wave - slot * ks;
  const int q = lane & 3, rg = lane >> 2;
  const int t = blockIdx.y;
  const int first_row = blockIdx.x * 16 * RG;  // RG groups of 16 rows share one staging of the activations
  const int nb = s.g.K / QK_K;
  const int chunk_elems = ks * QK_K, chunk_sb = ks * 8;
  const int64_t row_bytes = static_cast<int64_t>(nb) * GemvTraits<QT>::SUPER_BYTES;
  const int64_t expert_bytes = static_cast<int64_t>(s.g.N) * row_bytes;

  uint8_t* q8 = smem;
  float* xd = reinterpret_cast<float*>(q8 + TK * chunk_elems);
  float* xs = xd + TK * chunk_sb;
  int* s16 = reinterpret_cast<int*>(xs);
  float* red = gemv_has_mins(QT)  ? xs + TK * chunk_sb
             : (QT == GGML_Q6_K) ? reinterpret_cast<float*>(s16 + TK * chunk_sb * 2)
                                 : xs;                                  // [TK][ks][16 * RG]
  GemvArgs a = s.g;
  a.rows = s.top_k;
  a.x = static_cast<const uint8_t*>(s.g.x) + static_cast<int64_t>(t) * s.top_k * s.g.K * scalar_bytes(s.g.x_kind);
  ActTile tile{q8, xd, xs, s16, chunk_elems, chunk_sb};

  const int64_t e = slot < s.top_k ? s.selected[t * s.top_k + slot] : -1;
  const bool valid = e >= 0 && e < s.num_experts;
  const uint8_t* wexp = s.g.w + (valid ? e : 0) * expert_bytes;
  // routing weight of each slot (0 for a slot without a valid expert, whose dot is 0 too), fetched now and
  // kept in LDS: read from memory in the final sum, slot after slot, they were a chain of eight round trips
  float* rw = red + TK * ks * 16 * RG;
  if (kslice == 0 && lane == 0) rw[slot] = valid ? s.routing[t * s.top_k + slot] : 0.0f;

  float acc[RG];
#pragma unroll
  for (int g = 0; g < RG; ++g) acc[g] = 0.0f;
  for (int kc = 0; kc < nb; kc += ks) {
    Regs wr[RG];
    const int kb = kc + kslice;
    const bool live = valid && kb < nb;
#pragma unroll
    for (int g = 0; g < RG; ++g) {
      const int row = min(first_row + 16 * g + rg, s.g.N - 1);
      gemv_load_block<QT>(wexp + static_cast<int64_t>(row) * row_bytes +
                              static_cast<int64_t>(min(kb, nb - 1)) * GemvTraits<QT>::SUPER_BYTES, q, wr[g]);
    }
    if (kc > 0) __syncthreads();
    gemv_stage_activations<QT, TK>(a, kc, ks, q8, xd, xs, s16, chunk_elems, chunk_sb);
    __syncthreads();
#pragma unroll
    for (int g = 0; g < RG; ++g) {
      const BlockScales<QT> sc = gemv_block_scales<QT>(wr[g], q);
      const float term = gemv_block_term<QT>(wr[g], sc, q, tile, slot, kslice);
      acc[g] += live ? term : 0.0f;
    }
  }
#pragma unroll
  for (int g = 0; g < RG; ++g) {
    const float v = quad_sum(acc[g]);
    if (q == 0) red[(slot * ks + kslice) * 16 * RG + 16 * g + rg] = v;
  }
  __syncthreads();
  if (tid < 16 * RG && first_row + tid < s.g.N) {
    float total = 0.0f;
    for (int sl = 0; sl < s.top_k; ++sl) {
      float dot = 0.0f;
      for (int k = 0; k < ks; ++k) dot += red[(sl * ks + k) * 16 * RG + tid];
      total += rw[sl] * dot;
    }
    store_scalar(s.g.out, static_cast<int64_t>(t) * s.g.N + first_row + tid, total, s.g.out_kind);
  }
}

using SelFn = void (*)(SelArgs);
struct SelVariant {
  int qt, cb, mode, max_threads;
  SelFn fn;
  SelFn by_kind[2];   // float32 and bf16 activations
  SelFn silu_pair;    // single form over bf16(silu(gate) * up)
};
#define SEL_SINGLE_VARIANT(QT, CB)                                                                             \
  SelVariant{QT, CB, SEL_SINGLE, sel_max_threads<QT, CB>(), selected_gemv_kernel<QT, 1, CB, SEL_SINGLE>,          \
             {selected_gemv_kernel<QT, 1, CB, SEL_SINGLE, KIND_F32>, selected_gemv_kernel<QT, 1, CB, SEL_SINGLE, KIND_BF16>}, \
             selected_gemv_kernel<QT, 1, CB, SEL_SINGLE, KIND_SILU_BF16>}
#define SEL_VARIANTS(QT, CB)                                                                                   \
  SEL_SINGLE_VARIANT(QT, CB),                                                                                  \
  SelVariant{QT, CB, SEL_DUAL_SILU, sel_max_threads<QT, 2 * CB>(), selected_gemv_kernel<QT, 2, CB, SEL_DUAL_SILU>, \
             {selected_gemv_kernel<QT, 2, CB, SEL_DUAL_SILU, KIND_F32>, selected_gemv_kernel<QT, 2, CB, SEL_DUAL_SILU, KIND_BF16>}, \
             nullptr},                                                                                         \
  SelVariant{QT, CB, SEL_DUAL, sel_max_threads<QT, 2 * CB>(), selected_gemv_kernel<QT, 2, CB, SEL_DUAL>,          \
             {nullptr, nullptr}, nullptr}
// Q4_K and Q6_K experts take every form at every K; Q5_K and Q8_0 experts the two-matrix forms up to K = 4096
// (16 blocks per row: beyond that a lane would hold two matrices x five blocks of 17-20 registers)
const SelVariant kSel[] = {
    SEL_VARIANTS(GGML_Q4_K, 1), SEL_VARIANTS(GGML_Q4_K, 2), SEL_VARIANTS(GGML_Q4_K, 5),
    SEL_VARIANTS(GGML_Q6_K, 1), SEL_VARIANTS(GGML_Q6_K, 2), SEL_VARIANTS(GGML_Q6_K, 5),
    SEL_VARIANTS(GGML_Q5_K, 1), SEL_VARIANTS(GGML_Q5_K, 2), SEL_SINGLE_VARIANT(GGML_Q5_K, 5),
    SEL_VARIANTS(GGML_Q8_0, 1), SEL_VARIANTS(GGML_Q8_0, 2), SEL_SINGLE_VARIANT(GGML_Q8_0, 5),
};

int launch_selected(int qt, int mode, const void* x, int x_kind, const int64_t* selected, const float* routing,
                    const uint8_t* w_a, const uint8_t* w_b, void* out, int out_kind, int64_t x_rows, int64_t lanes,
                    int64_t num_experts, int64_t top_k, int64_t K, int64_t N, int round_mid, hipStream_t stream,
                    void* out_b = nullptr, const void* x_up = nullptr) {
  // q8_1 blocks as activations: the single and dual forms only (their staging reads them as they are);
  // x_up: the single form over bf16(silu(x) * x_up), both bf16
  const int max_x_kind = (mode == SEL_SINGLE || mode == SEL_DUAL) ? KIND_Q8_1 : KIND_F16;
  if (!x || !selected || !w_a || !out || x_rows <= 0 || lanes <= 0 || lanes > 65535 || num_experts <= 0 || K <= 0 ||
      (K % QK_K) != 0 || K > (1 << 20) || N <= 0 || N > (1 << 24) || x_kind < KIND_F32 || x_kind > max_x_kind ||
      out_kind < KIND_F32 || out_kind > KIND_F16 ||
      (qt != GGML_Q4_K && qt != GGML_Q5_K && qt != GGML_Q6_K && qt != GGML_Q8_0)) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  if (x_up && (mode != SEL_SINGLE || x_kind != KIND_BF16)) return static_cast<int>(hipErrorInvalidValue);
  if ((mode == SEL_DUAL_SILU || mode == SEL_DUAL) && !w_b) return static_cast<int>(hipErrorInvalidValue);
  if (mode == SEL_DUAL && !out_b) return static_cast<int>(hipErrorInvalidValue);
  if (mode == SEL_DOWN_SUM && (!routing || top_k <= 0 || top_k > 8 || lanes != x_rows * top_k)) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  if (mode != SEL_DOWN_SUM && (lanes % x_rows) != 0) return static_cast<int>(hipErrorInvalidValue);
  const int nb = static_cast<int>(K / QK_K);
  SelArgs s;
  s.g.x = x; s.g.w = w_a; s.g.out = out; s.g.x_kind = x_kind; s.g.out_kind = out_kind; s.g.rows = 1;
  s.g.K = static_cast<int>(K); s.g.N = static_cast<int>(N);
  s.g.x_up = x_up;
  s.w_b = w_b; s.out_b = out_b; s.selected = selected; s.routing = routing;
  s.x_rows = static_cast<int>(x_rows); s.lanes = static_cast<int>(lanes);
  s.num_experts = static_cast<int>(num_experts); s.top_k = static_cast<int>(top_k); s.round_mid = round_mid;
  s.pair_offset = 0;

  if (mode == SEL_DOWN_SUM) {
    // waves = 8 slots x ks K slices <= 16; one or two groups of 16 rows per workgroup, one as
    // long as the grid stays above ~2 workgroups per CU
    const int ks = nb >= 2 ? 2 : 1;
    // one workgroup per CU is resident (16 waves of ~80 registers): the fewest row groups per workgroup that
    // keep the grid within one round of 256 workgroups (measured, E=256 k=8 H=2048 I=512: T=4 8.4 us against
    // 12.7 with twice the workgroups, T=8 12.4 against 16.3)
    int rgn = 1;
    const int max_rgn = qt == GGML_Q5_K ? 2 : 4;   // four row groups of 20-register Q5_K blocks spill
    while (rgn < max_rgn && (N + 16 * rgn - 1) / (16 * rgn) * x_rows > 256) rgn <<= 1;   // 256 CUs
    s.g.ks = ks; s.g.nrg = rgn;
    const size_t lds = gemv_lds_bytes(qt, 8, 1, 1, ks, 1) + static_cast<size_t>(8) * ks * 16 * rgn * 4 + 8 * 4;
    if (lds > 64 * 1024) return static_cast<int>(hipErrorInvalidValue);
    const dim3 grid(static_cast<unsigned>((N + 16 * rgn - 1) / (16 * rgn)), static_cast<unsigned>(x_rows));
    const dim3 block(8 * ks * 64);
#define LAUNCH_DOWN(QT, RGN)                                                                                   \
  do {                                                                                                         \
    if (x_kind == KIND_F32) hipLaunchKernelGGL((selected_down_sum_kernel<QT, 8, RGN, KIND_F32>), grid, block, lds, stream, s); \
    else if (x_kind == KIND_BF16) hipLaunchKernelGGL((selected_down_sum_kernel<QT, 8, RGN, KIND_BF16>), grid, block, lds, stream, s); \
    else hipLaunchKernelGGL((selected_down_sum_kernel<QT, 8, RGN>), grid, block, lds, stream, s);                \
  } while (0)
#define LAUNCH_DOWN_QT(QT)                                                                                    \
  do {                                                                                                         \
    if (rgn == 4) LAUNCH_DOWN(QT, 4); else if (rgn == 2) LAUNCH_DOWN(QT, 2); else LAUNCH_DOWN(QT, 1);          \
  } while (0)
    if (qt == GGML_Q4_K) LAUNCH_DOWN_QT(GGML_Q4_K);
    else if (qt == GGML_Q5_K) { if (rgn == 2) LAUNCH_DOWN(GGML_Q5_K, 2); else LAUNCH_DOWN(GGML_Q5_K, 1); }
    else if (qt == GGML_Q6_K) LAUNCH_DOWN_QT(GGML_Q6_K);
    else LAUNCH_DOWN_QT(GGML_Q8_0);
#undef LAUNCH_DOWN_QT
#undef LAUNCH_DOWN
    return static_cast<int>(hipGetLastError());
  }

  // all of a row's blocks in flight at once when they fit 8 K slices, else chunks
  int ks, cb;
  if (nb <= 8) { ks = nb; cb = 1; }
  else if (nb <= 16) { ks = 8; cb = 2; }
  else { ks = 4; cb = 5; }
  const SelVariant* v = nullptr;
  for (const SelVariant& c : kSel)
    if (c.qt == qt && c.cb == cb && c.mode == mode) v = &c;
  if (!v) return static_cast<int>(hipErrorInvalidValue);
  const bool dual = mode == SEL_DUAL_SILU || mode == SEL_DUAL;
  const int r = dual ? 2 : 1;
  int nrg = v->max_threads / 64 / ks;
  if (nrg < 1) return static_cast<int>(hipErrorInvalidValue);
  const int rows_out_per_group = 16;
  // 16 rows per workgroup until the grid passes 2048 workgroups (measured, gate/up of 64 lanes x 512 rows, K = 2048:
  // 16.0 us at 16 rows per workgroup, 17.9 at 32, 18.5 with four K slices of two blocks)
  while (nrg > 1 && (N + nrg * rows_out_per_group - 1) / (nrg * rows_out_per_group) * lanes < 2048) nrg >>= 1;
  s.g.ks = ks; s.g.nrg = nrg;
  size_t lds = gemv_lds_bytes(qt, 1, r, cb, ks, nrg);
  if (mode == SEL_DUAL_SILU) {
    lds = (lds + 15) & ~static_cast<size_t>(15);
    s.pair_offset = static_cast<int>(lds);
    lds += 2 * nrg * 16 * 4;
  }
  if (lds > 64 * 1024) return static_cast<int>(hipErrorInvalidValue);
  const int rows_out = nrg * rows_out_per_group;
  const dim3 grid(static_cast<unsigned>((N + rows_out - 1) / rows_out), static_cast<unsigned>(lanes));
  const SelFn fn = x_up ? v->silu_pair
                   : ((x_kind == KIND_F32 || x_kind == KIND_BF16) && v->by_kind[x_kind]) ? v->by_kind[x_kind] : v->fn;
  if (!fn) return static_cast<int>(hipErrorInvalidValue);
  hipLaunchKernelGGL(fn, grid, dim3(ks * nrg * 64), lds, stream, s);
  return static_cast<int>(hipGetLastError());
}

// --------------------------------------------------------------------------
// grouped GEMV: compact rows (activations already gathered in expert-major order),
// every expert's weights read once per batch of 8 of its rows
// (kernels/hip_gfx1100/quant/gguf_q4_k_gemv.hip:378-450)
// --------------------------------------------------------------------------

struct GroupedArgs {
  GemvArgs g;                     // x [compact_rows, K], w [E, N, row_bytes], out [compact_rows, N]
  const int64_t* expert_start;    // [E + 1]
  int compact_rows;
};

// grid (row tiles of nrg*16 output rows, experts).  An expert's rows [start, end) are consecutive rows of x
// and out, so they are batch rows of the dense GEMV body; experts with one or two rows (a decode batch)
// take its batch-2 instantiation, the others walk their rows 8 at a time.
template <int QT, int CB>
__global__ void __launch_bounds__(512) grouped_gemv_kernel(GroupedArgs s) {
  extern __shared__ __align__(16) uint8_t smem[];
  const int e = blockIdx.y;
  const int64_t start = s.expert_start[e], end = s.expert_start[e + 1];
  if (start < 0 || end > s.compact_rows || start >= end) return;
  const int64_t row_bytes = static_cast<int64_t>(s.g.K / QK_K) * GemvTraits<QT>::SUPER_BYTES;
  const uint8_t* w = s.g.w + static_cast<int64_t>(e) * s.g.N * row_bytes;
  const int first_row = blockIdx.x * s.g.nrg * 16;
  GemvArgs a = s.g;
  const int64_t xb = act_row_bytes(s.g.x_kind, s.g.K), ob = static_cast<int64_t>(s.g.N) * scalar_bytes(s.g.out_kind);
  if (end - start <= 2) {
    a.rows = static_cast<int>(end - start);
    a.x = static_cast<const uint8_t*>(s.g.x) + start * xb;
    a.out = static_cast<uint8_t*>(s.g.out) + start * ob;
    gemv_workgroup<QT, 2, 1, CB>(a, w, first_row, smem);
    return;
  }
  for (int64_t base = start; base < end; base += 8) {
    a.rows = static_cast<int>(end - base < 8 ? end - base : 8);
    a.x = static_cast<const uint8_t*>(s.g.x) + base * xb;
    a.out = static_cast<uint8_t*>(s.g.out) + base * ob;
    if (base > start) __syncthreads();   // the staging area of the previous batch is still being read
    gemv_workgroup<QT, 8, 1, CB>(a, w, first_row, smem);
  }
}

int launch_grouped_gemv(int qt, const void* x, int x_kind, const int64_t* expert_start, const uint8_t* w, void* out,
                        int out_kind, int64_t compact_rows, int64_t num_experts, int64_t K, int64_t N,
                        hipStream_t stream) {
  if (!x || !expert_start || !w || !out || compact_rows <= 0 || compact_rows > 0x7FFFFFFF || num_experts <= 0 ||
      num_experts > 65535 || K <= 0 || (K % QK_K) != 0 || K > (1 << 20) || N <= 0 || N > (1 << 24) ||
      x_kind < KIND_F32 || x_kind > KIND_Q8_1 || out_kind < KIND_F32 || out_kind > KIND_F16 ||
      (qt != GGML_Q4_K && qt != GGML_Q5_K && qt != GGML_Q6_K && qt != GGML_Q8_0)) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  const int nb = static_cast<int>(K / QK_K);
  const int ks = nb >= 4 ? 4 : nb;
  const int per_wave = (nb + ks - 1) / ks;
  const int cb = per_wave >= 5 ? 5 : per_wave >= 2 ? 2 : 1;
  int nrg = 512 / 64 / ks;
  while (nrg > 1 && (N + nrg * 16 - 1) / (nrg * 16) < 8) nrg >>= 1;
  GroupedArgs s;
  s.g.x = x; s.g.w = w; s.g.out = out; s.g.x_kind = x_kind; s.g.out_kind = out_kind; s.g.rows = 8;
  s.g.K = static_cast<int>(K); s.g.N = static_cast<int>(N); s.g.ks = ks; s.g.nrg = nrg;
  s.expert_start = expert_start;
  s.compact_rows = static_cast<int>(compact_rows);
  const size_t lds = gemv_lds_bytes(qt, 8, 1, cb, ks, nrg);
  if (lds > 64 * 1024) return static_cast<int>(hipErrorInvalidValue);
  const dim3 grid(static_cast<unsigned>((N + nrg * 16 - 1) / (nrg * 16)), static_cast<unsigned>(num_experts));
  const dim3 block(ks * nrg * 64);
#define LAUNCH_GROUPED(QT)                                                                          \
  do {                                                                                              \
    if (cb == 1) hipLaunchKernelGGL((grouped_gemv_kernel<QT, 1>), grid, block, lds, stream, s);      \
    else if (cb == 2) hipLaunchKernelGGL((grouped_gemv_kernel<QT, 2>), grid, block, lds, stream, s); \
    else hipLaunchKernelGGL((grouped_gemv_kernel<QT, 5>), grid, block, lds, stream, s);              \
  } while (0)
  if (qt == GGML_Q4_K) LAUNCH_GROUPED(GGML_Q4_K);
  else if (qt == GGML_Q5_K) LAUNCH_GROUPED(GGML_Q5_K);
  else if (qt == GGML_Q6_K) LAUNCH_GROUPED(GGML_Q6_K);
  else LAUNCH_GROUPED(GGML_Q8_0);
#undef LAUNCH_GROUPED
  return static_cast<int>(hipGetLastError());
}

// --------------------------------------------------------------------------
// prefill: expert-grouped Q4_K x DS4 MMQ over 32-row tiles
// --------------------------------------------------------------------------

using MoeQ4 = Q4Tile<1, 2, 1, 4>;   // 32 compact rows x 256 columns, four waves side by side
using MoeQ5 = Q4Tile<1, 2, 1, 4, MMQ_Q5K_D4S4>;   // the same tile for Q5_K experts over D4S4 blocks

struct MoeMmqArgs {
  const uint8_t* xq;                 // DS4 (Q4_K) or D4S4 (Q5_K) blocks [source_rows, K/128]
  const int64_t* compact_to_source;  // [compact_rows] or null (compact row i reads source row i)
  const int64_t* expert_start_compact;
  const int64_t* expert_start_tiles; // row starts rounded up to 32 per expert
  const int64_t* tile_expert;        // [total_rows/32]
  const uint8_t* w_a;
  const uint8_t* w_b;
  void* out;                         // [compact_rows, Na + Nb]
  int out_kind;
  int compact_rows, source_rows, K, Na, Nb, num_experts;
  int64_t expert_stride_rows;
  int tiles_a;
};

template <class Tile>
__global__ void __launch_bounds__(Tile::THREADS, 2) moe_mmq_kernel(MoeMmqArgs a) {
  extern __shared__ __align__(16) uint8_t smem_raw[];
  typename Tile::Smem& s = *reinterpret_cast<typename Tile::Smem*>(smem_raw);
  int* src_row = reinterpret_cast<int*>(smem_raw + sizeof(typename Tile::Smem));

  const int tile_row = blockIdx.y;
  const int64_t e = a.tile_expert[tile_row];
  if (e < 0 || e >= a.num_experts) return;
  const bool use_b = static_cast<int>(blockIdx.x) >= a.tiles_a;
  const int n0 = (use_b ? blockIdx.x - a.tiles_a : blockIdx.x) * Tile::BN;
  const int local_n = use_b ? a.Nb : a.Na;
  const int64_t compact_base = a.expert_start_compact[e];
  const int64_t count = a.expert_start_compact[e + 1] - compact_base;
  const int64_t row0 = static_cast<int64_t>(tile_row) * Tile::BM - a.expert_start_tiles[e];
  const int64_t remaining = count - row0;
  if (row0 < 0 || remaining <= 0) return;
  const int valid_rows = remaining >= Tile::BM ? Tile::BM : static_cast<int>(remaining);
  const int64_t first_compact = compact_base + row0;
  if (compact_base < 0 || first_compact + valid_rows > a.compact_rows) return;

  const int steps = a.K / 128;
  const int64_t w_row_bytes = static_cast<int64_t>(a.K / QK_K) * Tile::W_BLOCK;
  const int64_t x_row_bytes = static_cast<int64_t>(steps) * Tile::A_BYTES;
  const int64_t stride_rows = a.expert_stride_rows > 0 ? a.expert_stride_rows : local_n;
  const uint8_t* w = (use_b ? a.w_b : a.w_a) + (e * stride_rows + n0) * w_row_bytes;   // the tile's first column

  if (threadIdx.x < Tile::BM) {
    const int64_t crow = first_compact + min(static_cast<int>(threadIdx.x), valid_rows - 1);
    int64_t src = a.compact_to_source ? a.compact_to_source[crow] : crow;
    src = src < 0 ? 0 : (src >= a.source_rows ? a.source_rows - 1 : src);
    src_row[threadIdx.x] = static_cast<int>(src);
  }
  __syncthreads();

  const int64_t out_stride = static_cast<int64_t>(a.Na) + a.Nb;
  const int col_base = (use_b ? a.Na : 0) + n0;
  Tile::template run<true, true>(
      a.xq, x_row_bytes, w, w_row_bytes, steps, s,
      [=](int row) { return static_cast<int64_t>(src_row[row]); },
      [=](int col) { return static_cast<int64_t>(min(col, local_n - 1 - n0)); },
      [=](int row, int col, float v) {
        if (row < valid_rows && n0 + col < local_n)
          store_scalar(a.out, (first_compact + row) * out_stride + col_base + col, v, a.out_kind);
      });
}

template <class Tile>
int launch_moe_mmq(const void* xq, const int64_t* compact_to_source, const int64_t* expert_start_compact,
                   const int64_t* expert_start_tiles, const int64_t* tile_expert, const uint8_t* w_a,
                   const uint8_t* w_b, void* out, int out_kind, int64_t compact_rows, int64_t source_rows, int64_t K,
                   int64_t Na, int64_t Nb, int64_t num_experts, int64_t total_rows, int64_t expert_stride_rows,
                   hipStream_t stream) {
  if (!xq || !expert_start_compact || !expert_start_tiles || !tile_expert || !w_a || !out || compact_rows <= 0 ||
      compact_rows > (1 << 24) || source_rows <= 0 || source_rows > (1 << 24) || K <= 0 || (K % QK_K) != 0 ||
      Na <= 0 || (Na % 32) != 0 || Nb < 0 || (Nb % 32) != 0 || (Nb > 0 && !w_b) || Na + Nb > (1 << 24) ||
      num_experts <= 0 || total_rows <= 0 || (total_rows % 32) != 0 || total_rows / 32 > 65535 ||
      expert_stride_rows < 0 || out_kind < KIND_F32 || out_kind > KIND_F16) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  if (sizeof(typename Tile::Smem) > 65536) {   // the LDS limit is raised at set-up
    const int rc = ensure_init();
    if (rc != static_cast<int>(hipSuccess)) return rc;
  }
  MoeMmqArgs a;
  a.xq = static_cast<const uint8_t*>(xq);
  a.compact_to_source = compact_to_source;
  a.expert_start_compact = expert_start_compact;
  a.expert_start_tiles = expert_start_tiles;
  a.tile_expert = tile_expert;
  a.w_a = w_a; a.w_b = w_b; a.out = out; a.out_kind = out_kind;
  a.compact_rows = static_cast<int>(compact_rows); a.source_rows = static_cast<int>(source_rows);
  a.K = static_cast<int>(K); a.Na = static_cast<int>(Na); a.Nb = static_cast<int>(Nb);
  a.num_experts = static_cast<int>(num_experts);
  a.expert_stride_rows = expert_stride_rows;
  a.tiles_a = static_cast<int>((Na + Tile::BN - 1) / Tile::BN);
  const int tiles_b = static_cast<int>((Nb + Tile::BN - 1) / Tile::BN);
  const dim3 grid(static_cast<unsigned>(a.tiles_a + tiles_b), static_cast<unsigned>(total_rows / 32));
  hipLaunchKernelGGL(moe_mmq_kernel<Tile>, grid, dim3(Tile::THREADS), sizeof(typename Tile::Smem) + Tile::BM * sizeof(int),
                     stream, a);
  return static_cast<int>(hipGetLastError());
}


// --------------------------------------------------------------------------
// prefill: expert-grouped Q6_K x D4S4 MMQ.  The tile engine of the dense GEMM over a map of 128-row tiles
// (expert per tile, built by the tile-map kernel with tile_rows = 128), rows gathered through
// compact_to_source; workgroup = (column tile of 64, row tile).
// --------------------------------------------------------------------------

struct MoeQ6Args {
  const uint8_t* xq;                 // D4S4 blocks [source_rows, K/128]
  const int64_t* compact_to_source;  // [compact_rows] or null (compact row i reads source row i)
  const int64_t* expert_start_compact;
  const int64_t* expert_start_tiles; // row starts rounded up to 128 per expert
  const int64_t* tile_expert;        // [total_rows/128]
  const uint8_t* w_a;
  const uint8_t* w_b;
  void* out;                         // [compact_rows, Na + Nb]
  int out_kind;
  int compact_rows, source_rows, K, Na, Nb, num_experts;
  int64_t expert_stride_rows;
  int tiles_a;
};

constexpr int MOE_Q6_COLS = 64;   // the 128-wide tile spills in this kernel (the row map on top of 243 registers)

// QT: GGML_Q6_K (the Q6_K tile engine) or GGML_Q8_0 (the Q8_0 one); the same tile shape and row map.
template <int QT>
struct MoeWideTile {
  using Smem = Q6Smem<MOE_Q6_COLS>;
  static constexpr int64_t row_bytes(int K) { return static_cast<int64_t>(K / QK_K) * Q6_K_BYTES; }
};
template <>
struct MoeWideTile<GGML_Q8_0> {
  using Smem = Q8Smem<MOE_Q6_COLS>;
  static constexpr int64_t row_bytes(int K) { return static_cast<int64_t>(K / 32) * Q8_0_BYTES; }
};

template <int QT>
__global__ void __launch_bounds__(Q6_THREADS, 2) moe_mmq_wide_kernel(MoeQ6Args a) {
  using Smem = typename MoeWideTile<QT>::Smem;
  extern __shared__ __align__(16) uint8_t smem_raw[];
  Smem& s = *reinterpret_cast<Smem*>(smem_raw);
  int* src_row = reinterpret_cast<int*>(smem_raw + sizeof(Smem));

  const int tile_row = blockIdx.y;
  const int64_t e = a.tile_expert[tile_row];
  if (e < 0 || e >= a.num_experts) return;
  const bool use_b = static_cast<int>(blockIdx.x) >= a.tiles_a;
  const int n0 = (use_b ? blockIdx.x - a.tiles_a : blockIdx.x) * MOE_Q6_COLS;
  const int local_n = use_b ? a.Nb : a.Na;
  const int64_t compact_base = a.expert_start_compact[e];
  const int64_t count = a.expert_start_compact[e + 1] - compact_base;
  const int64_t row0 = static_cast<int64_t>(tile_row) * Q6_BM - a.expert_start_tiles[e];
  const int64_t remaining = count - row0;
  if (row0 < 0 || remaining <= 0) return;
  const int valid_rows = remaining >= Q6_BM ? Q6_BM : static_cast<int>(remaining);
  const int64_t first_compact = compact_base + row0;
  if (compact_base < 0 || first_compact + valid_rows > a.compact_rows) return;

  const int steps = a.K / 128;
  const int64_t w_row_bytes = MoeWideTile<QT>::row_bytes(a.K);
  const int64_t x_row_bytes = static_cast<int64_t>(steps) * D4S4_BYTES;
  const int64_t stride_rows = a.expert_stride_rows > 0 ? a.expert_stride_rows : local_n;
  const uint8_t* w = (use_b ? a.w_b : a.w_a) + e * stride_rows * w_row_bytes;

  if (threadIdx.x < Q6_BM) {
    const int64_t crow = first_compact + min(static_cast<int>(threadIdx.x), valid_rows - 1);
    int64_t src = a.compact_to_source ? a.compact_to_source[crow] : crow;
    src = src < 0 ? 0 : (src >= a.source_rows ? a.source_rows - 1 : src);
    src_row[threadIdx.x] = static_cast<int>(src);
  }
  __syncthreads();

  const int64_t out_stride = static_cast<int64_t>(a.Na) + a.Nb;
  const int col_base = (use_b ? a.Na : 0) + n0;
  auto row_of = [=](int row) { return static_cast<int64_t>(src_row[row]); };
  auto col_of = [=](int col) { return static_cast<int64_t>(min(n0 + col, local_n - 1)); };
  auto emit = [=](int row, int col, float v) {
    if (row < valid_rows && n0 + col < local_n)
      store_scalar(a.out, (first_compact + row) * out_stride + col_base + col, v, a.out_kind);
  };
  if constexpr (QT == GGML_Q8_0) {
    q8_tile_run<false, MOE_Q6_COLS>(a.xq, x_row_bytes, w, w_row_bytes, steps, s, row_of, col_of, emit);
  } else {
    q6_tile_run<false, MOE_Q6_COLS>(a.xq, x_row_bytes, w, w_row_bytes, steps, s, row_of, col_of, emit);
  }
}

template <int QT>
int launch_moe_mmq_wide(const void* xq, const int64_t* compact_to_source, const int64_t* expert_start_compact,
                      const int64_t* expert_start_tiles, const int64_t* tile_expert, const uint8_t* w_a,
                      const uint8_t* w_b, void* out, int out_kind, int64_t compact_rows, int64_t source_rows, int64_t K,
                      int64_t Na, int64_t Nb, int64_t num_experts, int64_t total_rows, int64_t expert_stride_rows,
                      hipStream_t stream) {
  if (!xq || !expert_start_compact || !expert_start_tiles || !tile_expert || !w_a || !out || compact_rows <= 0 ||
      compact_rows > (1 << 24) || source_rows <= 0 || source_rows > (1 << 24) || K <= 0 ||
      (K % (QT == GGML_Q8_0 ? 128 : QK_K)) != 0 ||
      Na <= 0 || Nb < 0 || (Nb > 0 && !w_b) || Na + Nb > (1 << 24) || num_experts <= 0 || total_rows <= 0 ||
      (total_rows % Q6_BM) != 0 || total_rows / Q6_BM > 65535 || expert_stride_rows < 0 || out_kind < KIND_F32 ||
      out_kind > KIND_F16) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  MoeQ6Args a;
  a.xq = static_cast<const uint8_t*>(xq);
  a.compact_to_source = compact_to_source;
  a.expert_start_compact = expert_start_compact;
  a.expert_start_tiles = expert_start_tiles;
  a.tile_expert = tile_expert;
  a.w_a = w_a; a.w_b = w_b; a.out = out; a.out_kind = out_kind;
  a.compact_rows = static_cast<int>(compact_rows); a.source_rows = static_cast<int>(source_rows);
  a.K = static_cast<int>(K); a.Na = static_cast<int>(Na); a.Nb = static_cast<int>(Nb);
  a.num_experts = static_cast<int>(num_experts);
  a.expert_stride_rows = expert_stride_rows;
  a.tiles_a = static_cast<int>((Na + MOE_Q6_COLS - 1) / MOE_Q6_COLS);
  const int tiles_b = static_cast<int>((Nb + MOE_Q6_COLS - 1) / MOE_Q6_COLS);
  const dim3 grid(static_cast<unsigned>(a.tiles_a + tiles_b), static_cast<unsigned>(total_rows / Q6_BM));
  hipLaunchKernelGGL(moe_mmq_wide_kernel<QT>, grid, dim3(Q6_THREADS),
                     sizeof(typename MoeWideTile<QT>::Smem) + Q6_BM * sizeof(int), stream, a);
  return static_cast<int>(hipGetLastError());
}

// ---- MoE tail and the next RMSNorm ---------------------------------------------------
//
//   selected  = the token's routed sum, already rounded to bf16 (TAIL_AGGREGATE), or formed here from its slot rows
//               in slot order, acc = acc + value * weight in float32 with both roundings, then rounded to bf16
//               (TAIL_SLOTS: rows [token * rows + slot]; TAIL_GATHER: compact rows through lane_to_compact, a lane of
//               no expert contributes nothing)
//   residual' = bf16((residual + selected) + sigmoid(gate_logits[token * gate_stride]) * shared)
//   norm      = bf16((residual' * 1 / sqrt(mean(residual'^2) + eps)) * norm_weight)
//   (kernels/cpu_reference/ops.py:33-102; kernels/hip_gfx1100/fused/paro_combine.hip:452-482,575-700)
//
// One workgroup per token.  With features % 8 == 0 and features <= 8192 a thread owns up to four 8-value pieces,
// keeps residual' in registers between the two passes and moves 16 bytes per access, a group of up to eight slot
// rows in flight at a time; any other width takes one value per access and reads residual' back.
enum TailMode : int { TAIL_AGGREGATE = 0, TAIL_SLOTS = 1, TAIL_GATHER = 2 };

struct MoeTailArgs {
  const uint16_t* selected;
  const float* routing;
  const int64_t* lane_to_compact;
  const uint16_t* shared;
  const float* gate_logits;
  const uint16_t* residual;
  const float* norm_weight;
  uint16_t* norm_out;
  uint16_t* residual_out;
  int64_t features, gate_stride, compact_rows;
  int rows;
  float eps;
};

__device__ __forceinline__ void bf16x8_to_float(const uint4 p, float (&v)[8]) {
  const uint32_t w[4] = {p.x, p.y, p.z, p.w};
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    v[2 * e] = bf16_bits_to_float(w[e] & 0xFFFFu);
    v[2 * e + 1] = bf16_bits_to_float(w[e] >> 16);
  }
}

// A product and a sum that stay two roundings (the compiler contracts a * b + c into one otherwise, and HIP's
// __fmul_rn / __fadd_rn are the plain operators).
__device__ __forceinline__ float mul_rn(float a, float b) {
#pragma clang fp contract(off)
  return a * b;
}
__device__ __forceinline__ float add_rn(float a, float b) {
#pragma clang fp contract(off)
  return a + b;
}

__device__ __forceinline__ float tail_combine(float residual, float selected, float gate, float shared) {
  return bf16_bits_to_float(float_to_bf16_bits(add_rn(add_rn(residual, selected), mul_rn(gate, shared))));
}

// row of `selected` that slot s of the token reads, or -1
template <int MODE>
__device__ __forceinline__ int64_t tail_slot_row(const MoeTailArgs& a, int64_t lane) {
  if constexpr (MODE == TAIL_GATHER) {
    const int64_t c = a.lane_to_compact[lane];
    return (c >= 0 && c < a.compact_rows) ? c : -1;
  }
  return lane;
}

template <int MODE, bool VEC>
__global__ void __launch_bounds__(256) moe_tail_rmsnorm_kernel(MoeTailArgs a) {
  constexpr int NC = 4;   // 8-value pieces per thread: features <= 256 * 8 * NC
  const int64_t token = blockIdx.x;
  const int tid = threadIdx.x;
  const int64_t base = token * a.features;
  const float gate = 1.0f / (1.0f + expf(-a.gate_logits[token * a.gate_stride]));
  const int64_t lane0 = token * a.rows;
  float sumsq = 0.0f;
  float keep[NC][8];

  if constexpr (VEC) {
    const int64_t pieces = a.features >> 3;
#pragma unroll
    for (int i = 0; i < NC; ++i) {
      const int64_t col = (static_cast<int64_t>(tid) + i * 256) * 8;
      if (col >= pieces * 8) continue;
      float sel[8], res[8], sh[8];
      bf16x8_to_float(*reinterpret_cast<const uint4*>(a.residual + base + col), res);
      bf16x8_to_float(*reinterpret_cast<const uint4*>(a.shared + base + col), sh);
      if constexpr (MODE == TAIL_AGGREGATE) {
        bf16x8_to_float(*reinterpret_cast<const uint4*>(a.selected + base + col), sel);
      } else {
        float acc[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] = 0.0f;
        for (int s0 = 0; s0 < a.rows; s0 += 8) {
          int64_t row[8];
          float wgt[8];
          uint4 piece[8];
#pragma unroll
          for (int s = 0; s < 8; ++s) {
            const bool on = s0 + s < a.rows;
            row[s] = on ? tail_slot_row<MODE>(a, lane0 + s0 + s) : -1;
            wgt[s] = on ? a.routing[lane0 + s0 + s] : 0.0f;
          }
#pragma unroll
          for (int s = 0; s < 8; ++s)
            piece[s] = *reinterpret_cast<const uint4*>(a.selected + (row[s] >= 0 ? row[s] : 0) * a.features + col);
#pragma unroll
          for (int s = 0; s < 8; ++s) {
            if (row[s] < 0) continue;
            float v[8];
            bf16x8_to_float(piece[s], v);
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[e] = add_rn(acc[e], mul_rn(v[e], wgt[s]));
          }
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) sel[e] = bf16_bits_to_float(float_to_bf16_bits(acc[e]));
      }
      uint32_t packed[4];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float v = tail_combine(res[e], sel[e], gate, sh[e]);
        keep[i][e] = v;
        sumsq += v * v;
        const uint32_t bits = float_to_bits(v) >> 16;     // v is a bf16 value already
        packed[e >> 1] = (e & 1) ? (packed[e >> 1] | (bits << 16)) : bits;
      }
      *reinterpret_cast<uint4*>(a.residual_out + base + col) = make_uint4(packed[0], packed[1], packed[2], packed[3]);
    }
  } else {
    for (int64_t col = tid; col < a.features; col += 256) {
      float sel;
      if constexpr (MODE == TAIL_AGGREGATE) {
        sel = bf16_bits_to_float(a.selected[base + col]);
      } else {
        float acc = 0.0f;
        for (int s = 0; s < a.rows; ++s) {
          const int64_t row = tail_slot_row<MODE>(a, lane0 + s);
          if (row < 0) continue;
          acc = add_rn(acc, mul_rn(bf16_bits_to_float(a.selected[row * a.features + col]), a.routing[lane0 + s]));
        }
        sel = bf16_bits_to_float(float_to_bf16_bits(acc));
      }
      const float v = tail_combine(bf16_bits_to_float(a.residual[base + col]), sel, gate,
                                   bf16_bits_to_float(a.shared[base + col]));
      a.residual_out[base + col] = static_cast<uint16_t>(float_to_bits(v) >> 16);
      sumsq += v * v;
    }
  }

  __shared__ float wave_sum[4];
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) sumsq += __shfl_xor(sumsq, off);
  if ((tid & 63) == 0) wave_sum[tid >> 6] = sumsq;
  __syncthreads();
  const float total = (wave_sum[0] + wave_sum[1]) + (wave_sum[2] + wave_sum[3]);
  const float inv_rms = 1.0f / sqrtf(total / static_cast<float>(a.features) + a.eps);

  if constexpr (VEC) {
    const int64_t pieces = a.features >> 3;
#pragma unroll
    for (int i = 0; i < NC; ++i) {
      const int64_t col = (static_cast<int64_t>(tid) + i * 256) * 8;
      if (col >= pieces * 8) continue;
      const float4 w0 = *reinterpret_cast<const float4*>(a.norm_weight + col);
      const float4 w1 = *reinterpret_cast<const float4*>(a.norm_weight + col + 4);
      const float w[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
      uint32_t packed[4];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const uint32_t bits = float_to_bf16_bits(mul_rn(mul_rn(keep[i][e], inv_rms), w[e]));
        packed[e >> 1] = (e & 1) ? (packed[e >> 1] | (bits << 16)) : bits;
      }
      *reinterpret_cast<uint4*>(a.norm_out + base + col) = make_uint4(packed[0], packed[1], packed[2], packed[3]);
    }
  } else {
    for (int64_t col = tid; col < a.features; col += 256) {
      const float v = bf16_bits_to_float(a.residual_out[base + col]);   // this thread's own store
      a.norm_out[base + col] = float_to_bf16_bits(mul_rn(mul_rn(v, inv_rms), a.norm_weight[col]));
    }
  }
}

template <int MODE>
int launch_moe_tail(const uint16_t* selected, const float* routing, const int64_t* lane_to_compact,
                    const uint16_t* shared, const float* gate_logits, const uint16_t* residual,
                    const float* norm_weight, uint16_t* norm_out, uint16_t* residual_out, int64_t tokens, int64_t rows,
                    int64_t features, int64_t compact_rows, int64_t gate_stride, float eps, hipStream_t stream) {
  if (!selected || !shared || !gate_logits || !residual || !norm_weight || !norm_out || !residual_out || tokens <= 0 ||
      tokens > 0x7FFFFFFF || features <= 0 || gate_stride <= 0 || rows <= 0 || rows > 4096 ||
      (MODE != TAIL_AGGREGATE && !routing) || (MODE == TAIL_GATHER && (!lane_to_compact || compact_rows <= 0))) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  MoeTailArgs a;
  a.selected = selected; a.routing = routing; a.lane_to_compact = lane_to_compact; a.shared = shared;
  a.gate_logits = gate_logits; a.residual = residual; a.norm_weight = norm_weight; a.norm_out = norm_out;
  a.residual_out = residual_out; a.features = features; a.gate_stride = gate_stride; a.compact_rows = compact_rows;
  a.rows = static_cast<int>(rows); a.eps = eps;
  const uintptr_t align = reinterpret_cast<uintptr_t>(selected) | reinterpret_cast<uintptr_t>(shared) |
                          reinterpret_cast<uintptr_t>(residual) | reinterpret_cast<uintptr_t>(norm_weight) |
                          reinterpret_cast<uintptr_t>(norm_out) | reinterpret_cast<uintptr_t>(residual_out);
  const dim3 grid(static_cast<unsigned>(tokens));
  if ((features % 8) == 0 && features <= 8192 && (align & 15u) == 0) {
    hipLaunchKernelGGL((moe_tail_rmsnorm_kernel<MODE, true>), grid, dim3(256), 0, stream, a);
  } else {
    hipLaunchKernelGGL((moe_tail_rmsnorm_kernel<MODE, false>), grid, dim3(256), 0, stream, a);
  }
  return static_cast<int>(hipGetLastError());
}

// ---- router logits: logits[t, e] = hidden[t, :] . weight[e, :] in float32 (moe/router.hip:36-80) --------
//
// An unquantized product in front of the selection: hidden rows in float32, bf16 or fp16, weight rows in float32
// or in the 16-bit type of the hidden rows.  A wave owns 8 tokens x 4 weight rows; a lane walks K in pieces of 8
// values (16- and 32-byte loads), so a weight row is read once per 8 tokens and a hidden row once per 4 weight rows.
// Lanes are summed by a butterfly, the order of which differs from hipEngine's shared-memory tree: logits agree to
// float32 rounding, not bit for bit.
constexpr int RL_TOKENS = 8, RL_ROWS = 4, RL_WAVES = 4;

template <int KIND>
__device__ __forceinline__ void load8_as_float(const void* base, int64_t index, float (&v)[8]) {
  if constexpr (KIND == KIND_F32) {
    const float4 lo = *reinterpret_cast<const float4*>(static_cast<const float*>(base) + index);
    const float4 hi = *reinterpret_cast<const float4*>(static_cast<const float*>(base) + index + 4);
    v[0] = lo.x; v[1] = lo.y; v[2] = lo.z; v[3] = lo.w; v[4] = hi.x; v[5] = hi.y; v[6] = hi.z; v[7] = hi.w;
  } else {
    const uint4 p = *reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(base) + index);
    const uint32_t w[4] = {p.x, p.y, p.z, p.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      v[2 * e] = KIND == KIND_BF16 ? bf16_bits_to_float(w[e] & 0xFFFFu) : f16_bits_to_float(w[e] & 0xFFFFu);
      v[2 * e + 1] = KIND == KIND_BF16 ? bf16_bits_to_float(w[e] >> 16) : f16_bits_to_float(w[e] >> 16);
    }
  }
}

template <int HK, int WK>
__global__ void __launch_bounds__(64 * RL_WAVES) router_logits_kernel(const void* __restrict__ hidden,
                                                                      const void* __restrict__ weight,
                                                                      float* __restrict__ logits, int64_t tokens,
                                                                      int64_t hidden_size, int64_t num_rows, int64_t whole) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t row0 = (static_cast<int64_t>(blockIdx.x) * RL_WAVES + wave) * RL_ROWS;
  const int64_t tok0 = static_cast<int64_t>(blockIdx.y) * RL_TOKENS;
  if (row0 >= num_rows) return;     // whole waves leave; no workgroup barrier below
  float acc[RL_TOKENS][RL_ROWS];
#pragma unroll
  for (int t = 0; t < RL_TOKENS; ++t)
#pragma unroll
    for (int r = 0; r < RL_ROWS; ++r) acc[t][r] = 0.0f;
  // `whole`: the leading values of a row that go as 8-value pieces (16- and 32-byte loads); the rest one by one
  for (int64_t k = static_cast<int64_t>(lane) * 8; k < whole; k += 64 * 8) {
    float h[RL_TOKENS][8];
#pragma unroll
    for (int t = 0; t < RL_TOKENS; ++t) load8_as_float<HK>(hidden, min(tok0 + t, tokens - 1) * hidden_size + k, h[t]);
#pragma unroll
    for (int r = 0; r < RL_ROWS; ++r) {
      float w[8];
      load8_as_float<WK>(weight, min(row0 + r, num_rows - 1) * hidden_size + k, w);
#pragma unroll
      for (int t = 0; t < RL_TOKENS; ++t)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[t][r] = __builtin_fmaf(h[t][e], w[e], acc[t][r]);
    }
  }
  for (int64_t k = whole + lane; k < hidden_size; k += 64) {     // a row length that is not a multiple of 8
#pragma unroll
    for (int r = 0; r < RL_ROWS; ++r) {
      const float w = load_scalar(weight, min(row0 + r, num_rows - 1) * hidden_size + k, WK);
#pragma unroll
      for (int t = 0; t < RL_TOKENS; ++t)
        acc[t][r] = __builtin_fmaf(load_scalar(hidden, min(tok0 + t, tokens - 1) * hidden_size + k, HK), w, acc[t][r]);
    }
  }
#pragma unroll
  for (int t = 0; t < RL_TOKENS; ++t)
#pragma unroll
    for (int r = 0; r < RL_ROWS; ++r) {
      float v = acc[t][r];
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
      if (lane == 0 && tok0 + t < tokens && row0 + r < num_rows) logits[(tok0 + t) * num_rows + row0 + r] = v;
    }
}

// Decode batches (tokens <= 8): the four waves of a workgroup split K instead of the rows, so that a row of 2048 values
// is one 8-value piece per lane with every load of the workgroup in flight at once (the kernel above walks K in a
// loop of dependent round trips: 13.8 us at one token against the few microseconds of a 2 MB read).  TT tokens x
// RL_ROWS weight rows per workgroup; partial sums of the waves meet in LDS.
template <int HK, int WK, int TT>
__global__ void __launch_bounds__(64 * RL_WAVES) router_logits_decode_kernel(const void* __restrict__ hidden,
                                                                             const void* __restrict__ weight,
                                                                             float* __restrict__ logits, int64_t tokens,
                                                                             int64_t hidden_size, int64_t num_rows, int64_t whole) {
  __shared__ float part[RL_WAVES][TT][RL_ROWS];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t row0 = static_cast<int64_t>(blockIdx.x) * RL_ROWS;
  const int64_t tok0 = static_cast<int64_t>(blockIdx.y) * TT;
  float acc[TT][RL_ROWS];
#pragma unroll
  for (int t = 0; t < TT; ++t)
#pragma unroll
    for (int r = 0; r < RL_ROWS; ++r) acc[t][r] = 0.0f;
  for (int64_t k = (static_cast<int64_t>(wave) * 64 + lane) * 8; k < whole; k += 64 * RL_WAVES * 8) {
    float h[TT][8];
#pragma unroll
    for (int t = 0; t < TT; ++t) load8_as_float<HK>(hidden, min(tok0 + t, tokens - 1) * hidden_size + k, h[t]);
#pragma unroll
    for (int r = 0; r < RL_ROWS; ++r) {
      float w[8];
      load8_as_float<WK>(weight, min(row0 + r, num_rows - 1) * hidden_size + k, w);
#pragma unroll
      for (int t = 0; t < TT; ++t)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[t][r] = __builtin_fmaf(h[t][e], w[e], acc[t][r]);
    }
  }
  for (int64_t k = whole + wave * 64 + lane; k < hidden_size; k += 64 * RL_WAVES) {
#pragma unroll
    for (int r = 0; r < RL_ROWS; ++r) {
      const float w = load_scalar(weight, min(row0 + r, num_rows - 1) * hidden_size + k, WK);
#pragma unroll
      for (int t = 0; t < TT; ++t)
        acc[t][r] = __builtin_fmaf(load_scalar(hidden, min(tok0 + t, tokens - 1) * hidden_size + k, HK), w,
                                   acc[t][r]);
    }
  }
#pragma unroll
  for (int t = 0; t < TT; ++t)
#pragma unroll
    for (int r = 0; r < RL_ROWS; ++r) {
      float v = acc[t][r];
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
      if (lane == 0) part[wave][t][r] = v;
    }
  __syncthreads();
  if (threadIdx.x < TT * RL_ROWS) {
    const int t = threadIdx.x / RL_ROWS, r = threadIdx.x % RL_ROWS;
    if (tok0 + t < tokens && row0 + r < num_rows)
      logits[(tok0 + t) * num_rows + row0 + r] = (part[0][t][r] + part[1][t][r]) + (part[2][t][r] + part[3][t][r]);
  }
}

// Prefill batches with bf16 hidden rows: the product on the bf16 MFMA (v_mfma_f32_32x32x16_bf16).  A float32 weight is
// split into three bf16 parts that add up to it exactly (8 + 8 + 8 significant bits, each the truncation of what the
// parts before it leave), and the hidden values are bf16 already, so every product is exact in float32 and the sums
// have float32 accuracy: three MFMAs per 16 values instead of 16 x 32 x 32 FMAs (the kernel further up takes 73 us
// for 2048 tokens x 256 rows x 2048, most of it float32 FMAs and conversions).  A workgroup owns 32 tokens x 32
// rows; its four waves take a quarter of K each and meet in LDS.  Operands go from global memory straight into
// registers: lane (n = l % 32, g = l / 32) holds values 8g..8g+7 of the 16 of row n, on both sides alike.
typedef __bf16 rl_v8bf __attribute__((ext_vector_type(8)));
typedef float rl_v16f __attribute__((ext_vector_type(16)));

template <int WK>
__global__ void __launch_bounds__(256) router_logits_mfma_kernel(const uint16_t* __restrict__ hidden,
                                                                 const void* __restrict__ weight,
                                                                 float* __restrict__ logits, int64_t tokens,
                                                                 int64_t hidden_size, int64_t num_rows) {
  __shared__ float part[4][16][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n = lane & 31, g = lane >> 5;
  const int64_t row0 = static_cast<int64_t>(blockIdx.x) * 32, tok0 = static_cast<int64_t>(blockIdx.y) * 32;
  const int64_t k_per_wave = hidden_size / 4;                       // a multiple of 16
  const uint16_t* hrow = hidden + min(tok0 + n, tokens - 1) * hidden_size + wave * k_per_wave + 8 * g;
  const int64_t wbase = min(row0 + n, num_rows - 1) * hidden_size + wave * k_per_wave + 8 * g;
  // one accumulator per weight part: three independent MFMA chains instead of one of three times the length
  rl_v16f acc, acc_mid, acc_lo;
#pragma unroll
  for (int v = 0; v < 16; ++v) { acc[v] = 0.0f; acc_mid[v] = 0.0f; acc_lo[v] = 0.0f; }
#pragma unroll 4
  for (int64_t k = 0; k < k_per_wave; k += 16) {
    const uint4 hx = *reinterpret_cast<const uint4*>(hrow + k);
    const rl_v8bf a = __builtin_bit_cast(rl_v8bf, hx);
    if constexpr (WK == KIND_F32) {
      const float* wp = static_cast<const float*>(weight) + wbase + k;
      const float4 w0 = *reinterpret_cast<const float4*>(wp), w1 = *reinterpret_cast<const float4*>(wp + 4);
      const float w[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
      uint32_t hi[4], mid[4], lo[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        uint32_t p[3][2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const float x = w[2 * e + h];
          const uint32_t b0 = float_to_bits(x) & 0xFFFF0000u;
          const float r1 = x - bits_to_float(b0);
          const uint32_t b1 = float_to_bits(r1) & 0xFFFF0000u;
          const float r2 = r1 - bits_to_float(b1);
          p[0][h] = b0; p[1][h] = b1; p[2][h] = float_to_bits(r2) & 0xFFFF0000u;
        }
        hi[e] = (p[0][0] >> 16) | p[0][1];
        mid[e] = (p[1][0] >> 16) | p[1][1];
        lo[e] = (p[2][0] >> 16) | p[2][1];
      }
      acc_lo = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, __builtin_bit_cast(rl_v8bf, make_uint4(lo[0], lo[1], lo[2], lo[3])), acc_lo, 0, 0, 0);
      acc_mid = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, __builtin_bit_cast(rl_v8bf, make_uint4(mid[0], mid[1], mid[2], mid[3])), acc_mid, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, __builtin_bit_cast(rl_v8bf, make_uint4(hi[0], hi[1], hi[2], hi[3])), acc, 0, 0, 0);
    } else {
      const uint4 wx = *reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(weight) + wbase + k);
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, __builtin_bit_cast(rl_v8bf, wx), acc, 0, 0, 0);
    }
  }
#pragma unroll
  for (int v = 0; v < 16; ++v) part[wave][v][lane] = acc[v] + (acc_mid[v] + acc_lo[v]);   // small parts first
  __syncthreads();
  // lane holds weight row n and tokens 8*(v/4) + 4*g + v%4 of the tile
  for (int i = threadIdx.x; i < 16 * 64; i += 256) {
    const int v = i >> 6, l = i & 63;
    const int64_t tok = tok0 + 8 * (v >> 2) + 4 * (l >> 5) + (v & 3), row = row0 + (l & 31);
    if (tok < tokens && row < num_rows)
      logits[tok * num_rows + row] = (part[0][v][l] + part[1][v][l]) + (part[2][v][l] + part[3][v][l]);
  }
}

template <int HK, int WK>
int launch_router_logits(const void* hidden, const void* weight, float* logits, int64_t tokens, int64_t hidden_size,
                         int64_t num_rows, int64_t threads, hipStream_t stream) {
  const int64_t h_item = HK == KIND_F32 ? 4 : 2, w_item = WK == KIND_F32 ? 4 : 2;
  if (!hidden || !weight || !logits || tokens <= 0 || tokens > (1 << 24) || hidden_size <= 0 || num_rows <= 0 ||
      num_rows > (1 << 24) || !(threads == 64 || threads == 128 || threads == 256 || threads == 512) ||
      (reinterpret_cast<uintptr_t>(hidden) % h_item) != 0 || (reinterpret_cast<uintptr_t>(weight) % w_item) != 0) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  // the 16- and 32-byte loads want rows of 8-value pieces that start on their natural alignment; any other row
  // length or base address goes value by value (hipEngine's kernel takes any hidden_size: moe/router.hip:1016-1024)
  const bool vector_ok = ((hidden_size * h_item) % 16) == 0 && ((hidden_size * w_item) % 16) == 0 &&
                         (reinterpret_cast<uintptr_t>(hidden) & 15u) == 0 && (reinterpret_cast<uintptr_t>(weight) & 15u) == 0;
  const int64_t whole = vector_ok ? hidden_size & ~static_cast<int64_t>(7) : 0;
  if (tokens <= 8) {
    // one token, or groups of four tokens (eight tokens as one group measured 9.7 us against the 3 us of one token)
    const dim3 dgrid(static_cast<unsigned>((num_rows + RL_ROWS - 1) / RL_ROWS), tokens <= 4 ? 1u : 2u);
    if (tokens == 1) {
      hipLaunchKernelGGL((router_logits_decode_kernel<HK, WK, 1>), dgrid, dim3(64 * RL_WAVES), 0, stream, hidden, weight,
                         logits, tokens, hidden_size, num_rows, whole);
    } else {
      hipLaunchKernelGGL((router_logits_decode_kernel<HK, WK, 4>), dgrid, dim3(64 * RL_WAVES), 0, stream, hidden, weight,
                         logits, tokens, hidden_size, num_rows, whole);
    }
    return static_cast<int>(hipGetLastError());
  }
  if constexpr (HK == KIND_BF16 && (WK == KIND_F32 || WK == KIND_BF16)) {
    if (tokens >= 32 && (hidden_size % 64) == 0 && vector_ok) {
      const dim3 mgrid(static_cast<unsigned>((num_rows + 31) / 32), static_cast<unsigned>((tokens + 31) / 32));
      hipLaunchKernelGGL((router_logits_mfma_kernel<WK>), mgrid, dim3(256), 0, stream,
                         static_cast<const uint16_t*>(hidden), weight, logits, tokens, hidden_size, num_rows);
      return static_cast<int>(hipGetLastError());
    }
  }
  const dim3 grid(static_cast<unsigned>((num_rows + RL_WAVES * RL_ROWS - 1) / (RL_WAVES * RL_ROWS)),
                  static_cast<unsigned>((tokens + RL_TOKENS - 1) / RL_TOKENS));
  hipLaunchKernelGGL((router_logits_kernel<HK, WK>), grid, dim3(64 * RL_WAVES), 0, stream, hidden, weight, logits, tokens,
                     hidden_size, num_rows, whole);
  return static_cast<int>(hipGetLastError());
}

// ---- router: top-k experts of a row of logits and the softmax of their logits --------
//
// One wave per token.  Lane l keeps the experts l, l+64, ... (PER of them: 4 up to 256 experts, 16 up to 1024) in
// registers as 64-bit keys: the logit's bits mapped so that unsigned order is float order, above the complement of
// the expert index, so the largest key is the largest logit and, among equals, the lowest index; 0 stands for "no
// candidate" (past num_experts, NaN, a logit at or below the lowest float, a retired winner).  top_k times: every
// lane's largest key, the maximum over the wave (four DPP exchanges inside each row of 16 lanes, then the four rows
// through scalar registers: no trip through LDS, which made a round cost 0.85 us), and the owner retires its entry.
// The winners' logits sit in lanes 0..top_k-1 at the end, where the softmax over them is taken
// (max = the first winner, denominator floored at 1e-20: router.hip:628-715).
constexpr int ROUTER_MAX_PER_LANE = 16;
constexpr float ROUTER_LOWEST = -3.4028234663852886e38f;
constexpr int DPP_ROW_MIRROR = 0x140;   // lane i <-> lane 15-i inside each row of 16

struct RouterKey {
  uint32_t hi, lo;
};
__device__ __forceinline__ bool router_key_above(const RouterKey& a, const RouterKey& b) {
  return a.hi > b.hi || (a.hi == b.hi && a.lo > b.lo);
}
template <int CTRL>
__device__ __forceinline__ RouterKey router_key_dpp_max(const RouterKey& k) {
  const RouterKey o{static_cast<uint32_t>(dpp_i<CTRL>(static_cast<int>(k.hi))),
                    static_cast<uint32_t>(dpp_i<CTRL>(static_cast<int>(k.lo)))};
  return router_key_above(o, k) ? o : k;
}

template <int PER>
__global__ void __launch_bounds__(256) router_select_kernel(const float* __restrict__ logits,
                                                            int64_t* __restrict__ selected,
                                                            float* __restrict__ routing, int64_t tokens,
                                                            int64_t logits_stride, int num_experts, int top_k) {
  const int lane = threadIdx.x & 63;
  const int64_t token = static_cast<int64_t>(blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (token >= tokens) return;      // whole waves leave: the lane exchanges below see full waves
  const float* row = logits + token * logits_stride;
  RouterKey keys[PER];
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int ex = lane + 64 * i;
    const float f = ex < num_experts ? row[ex] : ROUTER_LOWEST;
    const uint32_t raw = float_to_bits(f);
    const uint32_t bits = raw == 0x80000000u ? 0u : raw;     // -0 and +0 are equal logits
    const bool candidate = f > ROUTER_LOWEST;     // false for NaN too
    keys[i].hi = candidate ? ((bits & 0x80000000u) ? ~bits : (bits | 0x80000000u)) : 0u;
    keys[i].lo = candidate ? ~static_cast<uint32_t>(ex) : 0u;
  }
  float mine = 0.0f;    // lane p < top_k: logit of the p-th winner
  for (int pos = 0; pos < top_k; ++pos) {
    RouterKey best = keys[0];
#pragma unroll
    for (int i = 1; i < PER; ++i) best = router_key_above(keys[i], best) ? keys[i] : best;
    best = router_key_dpp_max<DPP_QUAD_XOR1>(best);
    best = router_key_dpp_max<DPP_QUAD_XOR2>(best);
    best = router_key_dpp_max<DPP_ROW_HALF_MIRROR>(best);
    best = router_key_dpp_max<DPP_ROW_MIRROR>(best);       // every lane: the maximum of its row of 16
    RouterKey win{static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(best.hi), 0)),
                  static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(best.lo), 0))};
#pragma unroll
    for (int r = 1; r < 4; ++r) {
      const RouterKey o{static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(best.hi), 16 * r)),
                        static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(best.lo), 16 * r))};
      win = router_key_above(o, win) ? o : win;
    }
    const bool any = win.hi != 0u;
    const uint32_t wbits = (win.hi & 0x80000000u) ? (win.hi & 0x7FFFFFFFu) : ~win.hi;
    if (lane == pos) mine = any ? bits_to_float(wbits) : ROUTER_LOWEST;
    if (lane == 0) selected[token * top_k + pos] = any ? static_cast<int64_t>(~win.lo) : -1;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const bool gone = keys[i].hi == win.hi && keys[i].lo == win.lo;
      keys[i].hi = gone ? 0u : keys[i].hi;
      keys[i].lo = gone ? 0u : keys[i].lo;
    }
  }
  const float top = bits_to_float(static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(float_to_bits(mine)), 0)));
  const float ev = lane < top_k ? expf(mine - top) : 0.0f;
  float denom = 0.0f;
  for (int p = 0; p < top_k; ++p) {      // in position order, as the reference sums
    denom += bits_to_float(static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(float_to_bits(ev)), p)));
  }
  denom = fmaxf(denom, 1.0e-20f);
  if (lane < top_k) routing[token * top_k + lane] = ev / denom;
}
}  // namespace

// ---- routing index ------------------------------------------------------------

extern "C" int hipengine_qwen35_moe_group_compact_active(const int64_t* selected_experts, const float* routing_weights,
                                                         int64_t* expert_start, int64_t* active_experts,
                                                         int64_t* active_count, int64_t* sorted_lanes,
                                                         int64_t* sorted_experts, float* sorted_weights,
                                                         int64_t total_lanes, int64_t num_experts, hipStream_t stream) {
  return launch_compact(selected_experts, routing_weights, expert_start, active_experts, active_count, sorted_lanes,
                        sorted_experts, nullptr, sorted_weights, total_lanes, num_experts, 1, stream);
}

extern "C" int hipengine_qwen35_moe_group_compact_active_source_rows(
    const int64_t* selected_experts, const float* routing_weights, int64_t* expert_start, int64_t* active_experts,
    int64_t* active_count, int64_t* sorted_lanes, int64_t* compact_to_source, float* sorted_weights,
    int64_t total_lanes, int64_t num_experts, int64_t top_k, hipStream_t stream) {
  return launch_compact(selected_experts, routing_weights, expert_start, active_experts, active_count, sorted_lanes,
                        nullptr, compact_to_source, sorted_weights, total_lanes, num_experts, top_k, stream);
}

// The same index with the inverse (lane -> compact position, -1 for a lane of no expert) written by the same two
// launches, instead of a fill and a scatter after them.
extern "C" int hipengine_gfx950_moe_group_compact_index(
    const int64_t* selected_experts, const float* routing_weights, int64_t* expert_start, int64_t* active_experts,
    int64_t* active_count, int64_t* sorted_lanes, int64_t* compact_to_source, float* sorted_weights,
    int64_t* lane_to_compact, int64_t total_lanes, int64_t num_experts, int64_t top_k, hipStream_t stream) {
  if (!lane_to_compact) return static_cast<int>(hipErrorInvalidValue);
  return launch_compact(selected_experts, routing_weights, expert_start, active_experts, active_count, sorted_lanes,
                        nullptr, compact_to_source, sorted_weights, total_lanes, num_experts, top_k, stream,
                        lane_to_compact);
}

extern "C" int hipengine_qwen35_moe_mmq32_tile_map(const int64_t* expert_start_compact, int64_t* mmq_expert_start,
                                                   int64_t* tile_expert, int64_t* mmq_total_out, int64_t num_experts,
                                                   int64_t tile_capacity, hipStream_t stream) {
  return launch_tile_map(expert_start_compact, mmq_expert_start, tile_expert, mmq_total_out, num_experts, tile_capacity,
                         32, stream);
}

extern "C" int hipengine_qwen35_moe_group_count(const int64_t* selected_experts, int32_t* counts, int64_t total_lanes,
                                                int64_t num_experts, hipStream_t stream) {
  if (!selected_experts || !counts || total_lanes <= 0 || total_lanes > (1ll << 30) || num_experts <= 0) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  hipLaunchKernelGGL(moe_group_count_kernel, dim3(static_cast<unsigned>((total_lanes + 255) / 256)), dim3(256), 0,
                     stream, selected_experts, counts, total_lanes, num_experts);
  return static_cast<int>(hipGetLastError());
}

extern "C" int hipengine_qwen35_moe_group_prefix(const int32_t* counts, int32_t* padded_counts, int64_t* expert_start,
                                                 int64_t* total_padded, int64_t num_experts, int64_t pad_multiple,
                                                 hipStream_t stream) {
  if (!counts || !padded_counts || !expert_start || !total_padded || num_experts <= 0 || pad_multiple <= 0 ||
      num_experts > MAX_EXPERTS) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  hipLaunchKernelGGL(moe_group_prefix_kernel, dim3(1), dim3(1024), 0, stream, counts, padded_counts, expert_start,
                     total_padded, static_cast<int>(num_experts), pad_multiple);
  return static_cast<int>(hipGetLastError());
}

extern "C" int hipengine_qwen35_moe_gather_packed_hidden_lowp(const uint16_t* hidden_states, const int64_t* sorted_lanes,
                                                              uint16_t* packed_hidden, int64_t total_elements,
                                                              int64_t tokens, int64_t top_k, int64_t hidden_size,
                                                              hipStream_t stream) {
  if (!hidden_states || !sorted_lanes || !packed_hidden || total_elements <= 0 || tokens <= 0 || top_k <= 0 ||
      hidden_size <= 0 || (total_elements % hidden_size) != 0 || total_elements / hidden_size > 0x7FFFFFFF) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  const int64_t rows = total_elements / hidden_size;
  hipLaunchKernelGGL(moe_gather_rows_kernel, dim3(static_cast<unsigned>(rows)), dim3(256), 0, stream, hidden_states,
                     sorted_lanes, packed_hidden, rows, tokens, top_k, hidden_size);
  return static_cast<int>(hipGetLastError());
}

extern "C" int hipengine_qwen35_moe_group_scatter_gather_lowp(
    const uint16_t* hidden_states, const int64_t* selected_experts, const float* routing_weights,
    const int64_t* expert_start, int32_t* scatter_offsets, int64_t* sorted_lanes, int64_t* sorted_experts,
    float* sorted_weights, uint16_t* packed_hidden, int64_t total_lanes, int64_t num_experts, int64_t top_k,
    int64_t hidden_size, hipStream_t stream) {
  if (!hidden_states || !selected_experts || !routing_weights || !expert_start || !scatter_offsets || !sorted_lanes ||
      !sorted_experts || !sorted_weights || !packed_hidden || total_lanes <= 0 || total_lanes > 0x7FFFFFFF ||
      num_experts <= 0 || num_experts > MAX_EXPERTS || top_k <= 0 || hidden_size <= 0) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  // Rows of the outputs that no lane is scattered to (padding between experts) keep their contents, as in hipEngine.
  hipLaunchKernelGGL(moe_scatter_kernel, dim3(static_cast<unsigned>(num_experts)), dim3(1024), 0, stream,
                     selected_experts, routing_weights, expert_start, scatter_offsets, sorted_lanes, sorted_experts,
                     sorted_weights, total_lanes, hidden_states, packed_hidden, top_k, hidden_size);
  return static_cast<int>(hipGetLastError());
}

// hipEngine's "parallel" compaction variants produce the same arrays as its stable ones (one workgroup per expert,
// wave ballots keep ascending lane order: moe/group_scatter.hip:256-326), which is how the index is built here anyway.
extern "C" int hipengine_qwen35_moe_group_compact_active_parallel(
    const int64_t* selected_experts, const float* routing_weights, int64_t* expert_start, int64_t* active_experts,
    int64_t* active_count, int64_t* sorted_lanes, int64_t* sorted_experts, float* sorted_weights, int64_t total_lanes,
    int64_t num_experts, hipStream_t stream) {
  return hipengine_qwen35_moe_group_compact_active(selected_experts, routing_weights, expert_start, active_experts,
                                                   active_count, sorted_lanes, sorted_experts, sorted_weights,
                                                   total_lanes, num_experts, stream);
}

extern "C" int hipengine_qwen35_moe_group_compact_active_source_rows_parallel(
    const int64_t* selected_experts, const float* routing_weights, int64_t* expert_start, int64_t* active_experts,
    int64_t* active_count, int64_t* sorted_lanes, int64_t* compact_to_source, float* sorted_weights,
    int64_t total_lanes, int64_t num_experts, int64_t top_k, hipStream_t stream) {
  return hipengine_qwen35_moe_group_compact_active_source_rows(selected_experts, routing_weights, expert_start,
                                                               active_experts, active_count, sorted_lanes,
                                                               compact_to_source, sorted_weights, total_lanes,
                                                               num_experts, top_k, stream);
}

extern "C" int hipengine_qwen35_moe_group_compact_active_i32_parallel(
    const int32_t* selected_experts, const float* routing_weights, int64_t* expert_start, int64_t* active_experts,
    int64_t* active_count, int64_t* sorted_lanes, int64_t* sorted_experts, float* sorted_weights, int64_t total_lanes,
    int64_t num_experts, hipStream_t stream) {
  return launch_compact(selected_experts, routing_weights, expert_start, active_experts, active_count, sorted_lanes,
                        sorted_experts, nullptr, sorted_weights, total_lanes, num_experts, 1, stream);
}

extern "C" int hipengine_qwen35_moe_group_prefix_active(const int32_t* counts, int64_t* expert_start,
                                                        int64_t* active_experts, int64_t* active_count,
                                                        int64_t num_experts, hipStream_t stream) {
  if (!counts || !expert_start || !active_experts || !active_count || num_experts <= 0 || num_experts > MAX_EXPERTS) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  hipLaunchKernelGGL(moe_prefix_active_kernel, dim3(1), dim3(1024), 0, stream, counts, expert_start, active_experts,
                     active_count, static_cast<int>(num_experts));
  return static_cast<int>(hipGetLastError());
}

extern "C" int hipengine_qwen35_moe_group_scatter(const int64_t* selected_experts, const float* routing_weights,
                                                  const int64_t* expert_start, int32_t* scatter_offsets,
                                                  int64_t* sorted_lanes, int64_t* sorted_experts, float* sorted_weights,
                                                  int64_t total_lanes, int64_t num_experts,
                                                  bool include_routing_weights, hipStream_t stream) {
  if (!selected_experts || !expert_start || !scatter_offsets || !sorted_lanes || !sorted_experts ||
      (include_routing_weights && (!routing_weights || !sorted_weights)) || total_lanes <= 0 ||
      total_lanes > 0x7FFFFFFF || num_experts <= 0 || num_experts > MAX_EXPERTS) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  hipLaunchKernelGGL(moe_scatter_kernel, dim3(static_cast<unsigned>(num_experts)), dim3(1024), 0, stream,
                     selected_experts, routing_weights, expert_start, scatter_offsets, sorted_lanes, sorted_experts,
                     include_routing_weights ? sorted_weights : nullptr, total_lanes,
                     static_cast<const uint16_t*>(nullptr), static_cast<uint16_t*>(nullptr), static_cast<int64_t>(1),
                     static_cast<int64_t>(0));
  return static_cast<int>(hipGetLastError());
}

// The tile map for hipEngine's other tile heights: 16 rows (its WMMA tiles) and 64.
extern "C" int hipengine_qwen35_moe_wmma_tile_map(const int64_t* expert_start_compact, int64_t* wmma_expert_start,
                                                  int64_t* tile_expert, int64_t* wmma_total_out, int64_t num_experts,
                                                  int64_t tile_capacity, hipStream_t stream) {
  if (tile_capacity < 0) return static_cast<int>(hipErrorInvalidValue);
  return launch_tile_map(expert_start_compact, wmma_expert_start, tile_expert, wmma_total_out, num_experts,
                         tile_capacity, 16, stream);
}

extern "C" int hipengine_qwen35_moe_mmq64_tile_map(const int64_t* expert_start_compact, int64_t* mmq_expert_start,
                                                   int64_t* tile_expert, int64_t* mmq_total_out, int64_t num_experts,
                                                   int64_t tile_capacity, hipStream_t stream) {
  if (tile_capacity < 0) return static_cast<int>(hipErrorInvalidValue);
  return launch_tile_map(expert_start_compact, mmq_expert_start, tile_expert, mmq_total_out, num_experts,
                         tile_capacity, 64, stream);
}

extern "C" int hipengine_gfx950_moe_lane_to_compact(const int64_t* sorted_lanes, int64_t* lane_to_compact,
                                                    int64_t compact_rows, int64_t total_lanes, hipStream_t stream) {
  if (!sorted_lanes || !lane_to_compact || compact_rows <= 0 || total_lanes <= 0) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  hipLaunchKernelGGL(moe_fill_i64_kernel, dim3(static_cast<unsigned>((total_lanes + 255) / 256)), dim3(256), 0, stream,
                     lane_to_compact, total_lanes, static_cast<int64_t>(-1));
  hipLaunchKernelGGL(moe_invert_kernel, dim3(static_cast<unsigned>((compact_rows + 255) / 256)), dim3(256), 0, stream,
                     sorted_lanes, lane_to_compact, compact_rows, total_lanes);
  return static_cast<int>(hipGetLastError());
}

// ---- elementwise steps ----------------------------------------------------------

extern "C" int hipengine_gfx950_moe_silu_mul(const void* gate_up, void* out, int64_t rows, int64_t inter, int in_kind,
                                             int out_kind, hipStream_t stream) {
  if (!gate_up || !out || rows <= 0 || inter <= 0 || in_kind < KIND_F32 || in_kind > KIND_F16 || out_kind < KIND_F32 ||
      out_kind > KIND_F16 || rows * inter > (1ll << 40)) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  hipLaunchKernelGGL(moe_silu_mul_kernel, dim3(static_cast<unsigned>((rows * inter + 255) / 256)), dim3(256), 0, stream,
                     gate_up, out, rows, inter, in_kind, out_kind);
  return static_cast<int>(hipGetLastError());
}

// The MoE tail with the next layer's RMSNorm (bf16 rows, float32 norm weight) for a routed sum that is already
// formed and rounded, for slot rows [tokens * rows_per_token, features] with their routing weights, and for compact
// rows gathered through lane_to_compact.
extern "C" int hipengine_shared_gate_combine_residual_rmsnorm_gguf_bf16_out(
    const uint16_t* selected, const uint16_t* shared, const float* gate_logits, const uint16_t* residual,
    const float* norm_weight, uint16_t* norm_out, uint16_t* residual_out, int64_t tokens, int64_t features,
    int64_t gate_stride, float eps, hipStream_t stream) {
  return launch_moe_tail<TAIL_AGGREGATE>(selected, nullptr, nullptr, shared, gate_logits, residual, norm_weight, norm_out,
                                         residual_out, tokens, 1, features, 0, gate_stride, eps, stream);
}

extern "C" int hipengine_weighted_sum_shared_gate_combine_residual_rmsnorm_gguf_bf16_out(
    const uint16_t* selected_values, const float* routing_weights, const uint16_t* shared, const float* gate_logits,
    const uint16_t* residual, const float* norm_weight, uint16_t* norm_out, uint16_t* residual_out, int64_t tokens,
    int64_t rows_per_token, int64_t features, int64_t gate_stride, float eps, hipStream_t stream) {
  return launch_moe_tail<TAIL_SLOTS>(selected_values, routing_weights, nullptr, shared, gate_logits, residual,
                                     norm_weight, norm_out, residual_out, tokens, rows_per_token, features, 0,
                                     gate_stride, eps, stream);
}

extern "C" int hipengine_gfx950_moe_gather_tail_rmsnorm_bf16(
    const uint16_t* down, const int64_t* lane_to_compact, const float* routing_weights, const uint16_t* shared,
    const float* gate_logits, const uint16_t* residual, const float* norm_weight, uint16_t* norm_out,
    uint16_t* residual_out, int64_t tokens, int64_t top_k, int64_t features, int64_t compact_rows, int64_t gate_stride,
    float eps, hipStream_t stream) {
  return launch_moe_tail<TAIL_GATHER>(down, routing_weights, lane_to_compact, shared, gate_logits, residual, norm_weight,
                                      norm_out, residual_out, tokens, top_k, features, compact_rows, gate_stride, eps,
                                      stream);
}

extern "C" int hipengine_gfx950_moe_weighted_gather_sum(const void* down, const int64_t* lane_to_compact,
                                                        const float* routing_weights, void* out, int64_t tokens,
                                                        int64_t top_k, int64_t hidden, int64_t compact_rows,
                                                        int in_kind, int out_kind, hipStream_t stream) {
  if (!down || !lane_to_compact || !routing_weights || !out || tokens <= 0 || tokens > 65535 || top_k <= 0 ||
      hidden <= 0 || compact_rows <= 0 || in_kind < KIND_F32 || in_kind > KIND_F16 || out_kind < KIND_F32 ||
      out_kind > KIND_F16) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  if ((hidden % 8) == 0 && top_k <= 8 && ((reinterpret_cast<uintptr_t>(down) | reinterpret_cast<uintptr_t>(out)) & 15u) == 0) {
    const dim3 grid(static_cast<unsigned>((hidden / 8 + 255) / 256), static_cast<unsigned>(tokens));
    const int k = static_cast<int>(top_k);
    if (in_kind == KIND_F32) {
      hipLaunchKernelGGL(moe_weighted_gather8_kernel<KIND_F32>, grid, dim3(256), 0, stream, down, lane_to_compact,
                         routing_weights, out, tokens, k, hidden, compact_rows, out_kind);
    } else if (in_kind == KIND_BF16) {
      hipLaunchKernelGGL(moe_weighted_gather8_kernel<KIND_BF16>, grid, dim3(256), 0, stream, down, lane_to_compact,
                         routing_weights, out, tokens, k, hidden, compact_rows, out_kind);
    } else {
      hipLaunchKernelGGL(moe_weighted_gather8_kernel<KIND_F16>, grid, dim3(256), 0, stream, down, lane_to_compact,
                         routing_weights, out, tokens, k, hidden, compact_rows, out_kind);
    }
    return static_cast<int>(hipGetLastError());
  }
  hipLaunchKernelGGL(moe_weighted_gather_kernel, dim3(static_cast<unsigned>((hidden + 255) / 256),
                                                      static_cast<unsigned>(tokens)),
                     dim3(256), 0, stream, down, lane_to_compact, routing_weights, out, tokens, top_k, hidden,
                     compact_rows, in_kind, out_kind);
  return static_cast<int>(hipGetLastError());
}

// ---- decode ---------------------------------------------------------------------

extern "C" int hipengine_gguf_q4_k_selected_gemv_bf16_bf16_out(const uint16_t* x, const int64_t* selected,
                                                               const uint8_t* qweight, uint16_t* out, int64_t x_rows,
                                                               int64_t rows, int64_t num_experts, int64_t in_features,
                                                               int64_t out_features, int64_t threads,
                                                               hipStream_t stream) {
  (void)threads;
  return launch_selected(GGML_Q4_K, SEL_SINGLE, x, KIND_BF16, selected, nullptr, qweight, nullptr, out, KIND_BF16,
                         x_rows, rows, num_experts, 1, in_features, out_features, 0, stream);
}

// The same for Q5_K / Q6_K / Q8_0 experts, and their down projection over bf16(silu(gate) * up) formed from the
// gate and up rows while the activations are staged (gguf_k_gemv.hip:5586-5599, kernel :1813-1866).
#define DEFINE_SELECTED_K(QNAME, QT)                                                                                 \
  extern "C" int hipengine_gguf_##QNAME##_selected_gemv_bf16_bf16_out(                                               \
      const uint16_t* x, const int64_t* selected, const uint8_t* qweight, uint16_t* out, int64_t x_rows,             \
      int64_t rows, int64_t num_experts, int64_t in_features, int64_t out_features, int64_t /*threads*/,            \
      hipStream_t stream) {                                                                                          \
    return launch_selected(QT, SEL_SINGLE, x, KIND_BF16, selected, nullptr, qweight, nullptr, out, KIND_BF16, x_rows, \
                           rows, num_experts, 1, in_features, out_features, 0, stream);                              \
  }                                                                                                                  \
  extern "C" int hipengine_gguf_##QNAME##_selected_silu_gemv_bf16_bf16_out(                                          \
      const uint16_t* gate, const uint16_t* up, const int64_t* selected, const uint8_t* qweight, uint16_t* out,      \
      int64_t x_rows, int64_t rows, int64_t num_experts, int64_t in_features, int64_t out_features,                  \
      int64_t /*threads*/, hipStream_t stream) {                                                                     \
    if (!up) return static_cast<int>(hipErrorInvalidValue);                                                          \
    return launch_selected(QT, SEL_SINGLE, gate, KIND_BF16, selected, nullptr, qweight, nullptr, out, KIND_BF16,     \
                           x_rows, rows, num_experts, 1, in_features, out_features, 0, stream, nullptr, up);         \
  }
DEFINE_SELECTED_K(q5_k, GGML_Q5_K)
DEFINE_SELECTED_K(q6_k, GGML_Q6_K)
DEFINE_SELECTED_K(q8_0, GGML_Q8_0)

extern "C" int hipengine_gguf_q4_k_selected_dual_silu_gemv_bf16_bf16_out(
    const uint16_t* x, const int64_t* selected, const uint8_t* qweight_a, const uint8_t* qweight_b, uint16_t* out,
    int64_t x_rows, int64_t rows, int64_t num_experts, int64_t in_features, int64_t out_features, int64_t threads,
    hipStream_t stream) {
  (void)threads;
  return launch_selected(GGML_Q4_K, SEL_DUAL_SILU, x, KIND_BF16, selected, nullptr, qweight_a, qweight_b, out,
                         KIND_BF16, x_rows, rows, num_experts, 1, in_features, out_features, 1, stream);
}

// out_a[lane] = W_a[selected[lane]] . x_row, out_b[lane] = W_b[selected[lane]] . x_row in one pass
// (gguf_q4_k_gemv.hip:2732-2749), and the same over pre-quantized 36-byte q8_1 activation rows (:2864-2892).
extern "C" int hipengine_gguf_q4_k_selected_dual_gemv_bf16_bf16_out(
    const uint16_t* x, const int64_t* selected, const uint8_t* qweight_a, const uint8_t* qweight_b, uint16_t* out_a,
    uint16_t* out_b, int64_t x_rows, int64_t rows, int64_t num_experts, int64_t in_features, int64_t out_features,
    int64_t threads, hipStream_t stream) {
  (void)threads;
  return launch_selected(GGML_Q4_K, SEL_DUAL, x, KIND_BF16, selected, nullptr, qweight_a, qweight_b, out_a, KIND_BF16,
                         x_rows, rows, num_experts, 1, in_features, out_features, 0, stream, out_b);
}

extern "C" int hipengine_gguf_q4_k_selected_dual_gemv_q8_1_dp4a_bf16_bf16_out(
    const void* xq, const int64_t* selected, const uint8_t* qweight_a, const uint8_t* qweight_b, uint16_t* out_a,
    uint16_t* out_b, int64_t x_rows, int64_t rows, int64_t num_experts, int64_t in_features, int64_t out_features,
    int64_t threads, hipStream_t stream) {
  (void)threads;
  return launch_selected(GGML_Q4_K, SEL_DUAL, xq, KIND_Q8_1, selected, nullptr, qweight_a, qweight_b, out_a, KIND_BF16,
                         x_rows, rows, num_experts, 1, in_features, out_features, 0, stream, out_b);
}

// Routed down projection with the weighted sum over a token's experts fused ("weighted_down" call kind,
// loading/gguf_selected_contract.py:50-54,305-315; argument list of
// hipengine_gguf_iq4_xs_weighted_selected_down_bf16_bf16_out, gguf_iq_gemv.hip:2276-2288).
#define DEFINE_WEIGHTED_DOWN(QNAME, QT)                                                                              \
  extern "C" int hipengine_gguf_##QNAME##_weighted_selected_down_bf16_bf16_out(                                      \
      const uint16_t* x, const int64_t* selected, const float* routing_weights, const uint8_t* qweight, uint16_t* out, \
      int64_t tokens, int64_t top_k, int64_t num_experts, int64_t in_features, int64_t out_features, int64_t threads, \
      hipStream_t stream) {                                                                                          \
    (void)threads;                                                                                                   \
    if (tokens <= 0 || top_k <= 0 || tokens * top_k > 65535) return static_cast<int>(hipErrorInvalidValue);          \
    return launch_selected(QT, SEL_DOWN_SUM, x, KIND_BF16, selected, routing_weights, qweight, nullptr, out,         \
                           KIND_BF16, tokens, tokens * top_k, num_experts, top_k, in_features, out_features, 0,      \
                           stream);                                                                                  \
  }
DEFINE_WEIGHTED_DOWN(q4_k, GGML_Q4_K)
DEFINE_WEIGHTED_DOWN(q6_k, GGML_Q6_K)

// Grouped GEMV over gathered compact rows (gguf_q4_k_gemv.hip:2634-2669).
extern "C" int hipengine_gguf_q4_k_selected_grouped_prefill_compact_rowbatch8_bf16_bf16_out(
    const void* x, const void* expert_start, const void* qweight, void* out, int64_t compact_rows, int64_t num_experts,
    int64_t in_features, int64_t out_features, hipStream_t stream) {
  return launch_grouped_gemv(GGML_Q4_K, x, KIND_BF16, static_cast<const int64_t*>(expert_start),
                             static_cast<const uint8_t*>(qweight), out, KIND_BF16, compact_rows, num_experts,
                             in_features, out_features, stream);
}

// The same for expert weights of any of the four block types and any activation / output kind.
extern "C" int hipengine_gfx950_gguf_grouped_gemv(int32_t ggml_type, const void* x, int32_t x_kind,
                                                  const int64_t* expert_start, const uint8_t* qweight, void* out,
                                                  int32_t out_kind, int64_t compact_rows, int64_t num_experts,
                                                  int64_t in_features, int64_t out_features, hipStream_t stream) {
  return launch_grouped_gemv(ggml_type, x, x_kind, expert_start, qweight, out, out_kind, compact_rows, num_experts,
                             in_features, out_features, stream);
}

extern "C" int hipengine_gfx950_gguf_selected_gemv(int32_t ggml_type, int32_t mode, const void* x, int32_t x_kind,
                                                   const int64_t* selected, const float* routing_weights,
                                                   const uint8_t* qweight_a, const uint8_t* qweight_b, void* out,
                                                   int32_t out_kind, int64_t x_rows, int64_t lanes,
                                                   int64_t num_experts, int64_t top_k, int64_t in_features,
                                                   int64_t out_features, int32_t round_mid, hipStream_t stream) {
  if (mode < SEL_SINGLE || mode > SEL_DOWN_SUM) return static_cast<int>(hipErrorInvalidValue);
  return launch_selected(ggml_type, mode, x, x_kind, selected, routing_weights, qweight_a, qweight_b, out, out_kind,
                         x_rows, lanes, num_experts, top_k, in_features, out_features, round_mid, stream);
}

// ---- prefill ----------------------------------------------------------------------

extern "C" int hipengine_gguf_q4_k_selected_dual_q8_1_ds4_mmq32_prefill_compact32_bf16_bf16_out(
    const void* x_q8, const int64_t* compact_to_source, const int64_t* expert_start_compact,
    const int64_t* expert_start_mmq32, const int64_t* tile_expert, const uint8_t* qweight_a, const uint8_t* qweight_b,
    uint16_t* out, int64_t compact_rows, int64_t in_features, int64_t out_features_a, int64_t out_features_b,
    int64_t num_experts, int64_t mmq_total_rows, int64_t expert_stride_rows, hipStream_t stream) {
  if (!compact_to_source) return static_cast<int>(hipErrorInvalidValue);
  // As in hipEngine, the activation rows are addressed through compact_to_source only and the source row count is
  // not part of this signature: no upper clamp (lanes dropped from the index can leave fewer compact rows than
  // there are tokens, and a clamp to the compact row count would then redirect the last tokens).
  return launch_moe_mmq<MoeQ4>(x_q8, compact_to_source, expert_start_compact, expert_start_mmq32, tile_expert, qweight_a,
                        qweight_b, out, KIND_BF16, compact_rows, 1 << 24, in_features, out_features_a,
                        out_features_b, num_experts, mmq_total_rows, expert_stride_rows, stream);
}

// hipEngine's 32 x 128 tile variant of the same GEMM (gguf_q4_k_q8_1_selected_prefill.hip:7510-7548): no expert
// stride argument.
extern "C" int hipengine_gguf_q4_k_selected_dual_q8_1_ds4_mmq32x128_prefill_compact32_bf16_bf16_out(
    const void* x_q8, const int64_t* compact_to_source, const int64_t* expert_start_compact,
    const int64_t* expert_start_mmq32, const int64_t* tile_expert, const uint8_t* qweight_a, const uint8_t* qweight_b,
    uint16_t* out, int64_t compact_rows, int64_t in_features, int64_t out_features_a, int64_t out_features_b,
    int64_t num_experts, int64_t mmq_total_rows, hipStream_t stream) {
  return hipengine_gguf_q4_k_selected_dual_q8_1_ds4_mmq32_prefill_compact32_bf16_bf16_out(
      x_q8, compact_to_source, expert_start_compact, expert_start_mmq32, tile_expert, qweight_a, qweight_b, out,
      compact_rows, in_features, out_features_a, out_features_b, num_experts, mmq_total_rows, 0, stream);
}

extern "C" int hipengine_gfx950_gguf_q4_k_grouped_mmq(const void* x_q8, const int64_t* compact_to_source,
                                                      const int64_t* expert_start_compact,
                                                      const int64_t* expert_start_mmq32, const int64_t* tile_expert,
                                                      const uint8_t* qweight_a, const uint8_t* qweight_b, void* out,
                                                      int32_t out_kind, int64_t compact_rows, int64_t source_rows,
                                                      int64_t in_features, int64_t out_features_a,
                                                      int64_t out_features_b, int64_t num_experts,
                                                      int64_t mmq_total_rows, int64_t expert_stride_rows,
                                                      hipStream_t stream) {
  return launch_moe_mmq<MoeQ4>(x_q8, compact_to_source, expert_start_compact, expert_start_mmq32, tile_expert, qweight_a,
                        qweight_b, out, out_kind, compact_rows, source_rows, in_features, out_features_a,
                        out_features_b, num_experts, mmq_total_rows, expert_stride_rows, stream);
}

// The same for Q5_K expert weights over D4S4 activation blocks (the 32-row tile map).
extern "C" int hipengine_gfx950_gguf_q5_k_grouped_mmq(const void* x_d4s4, const int64_t* compact_to_source,
                                                      const int64_t* expert_start_compact,
                                                      const int64_t* expert_start_mmq32, const int64_t* tile_expert,
                                                      const uint8_t* qweight_a, const uint8_t* qweight_b, void* out,
                                                      int32_t out_kind, int64_t compact_rows, int64_t source_rows,
                                                      int64_t in_features, int64_t out_features_a,
                                                      int64_t out_features_b, int64_t num_experts,
                                                      int64_t mmq_total_rows, int64_t expert_stride_rows,
                                                      hipStream_t stream) {
  return launch_moe_mmq<MoeQ5>(x_d4s4, compact_to_source, expert_start_compact, expert_start_mmq32, tile_expert,
                               qweight_a, qweight_b, out, out_kind, compact_rows, source_rows, in_features,
                               out_features_a, out_features_b, num_experts, mmq_total_rows, expert_stride_rows, stream);
}

// The expert-grouped MMQ for Q6_K expert weights over D4S4 activation blocks: out[compact row, :] =
// [W_a[e] | W_b[e]] x, e the expert that owns the compact row.  The tile map is one of 128-row tiles
// (hipengine_gfx950_moe_tile_map with tile_rows = 128): total_rows a multiple of 128.
extern "C" int hipengine_gfx950_gguf_q6_k_grouped_mmq(const void* x_d4s4, const int64_t* compact_to_source,
                                                      const int64_t* expert_start_compact,
                                                      const int64_t* expert_start_tiles, const int64_t* tile_expert,
                                                      const uint8_t* qweight_a, const uint8_t* qweight_b, void* out,
                                                      int32_t out_kind, int64_t compact_rows, int64_t source_rows,
                                                      int64_t in_features, int64_t out_features_a,
                                                      int64_t out_features_b, int64_t num_experts,
                                                      int64_t total_rows, int64_t expert_stride_rows,
                                                      hipStream_t stream) {
  return launch_moe_mmq_wide<GGML_Q6_K>(x_d4s4, compact_to_source, expert_start_compact, expert_start_tiles,
                                        tile_expert, qweight_a, qweight_b, out, out_kind, compact_rows, source_rows,
                                        in_features, out_features_a, out_features_b, num_experts, total_rows,
                                        expert_stride_rows, stream);
}

// The same for Q8_0 expert weights (34-byte blocks): in_features a multiple of 128.
extern "C" int hipengine_gfx950_gguf_q8_0_grouped_mmq(const void* x_d4s4, const int64_t* compact_to_source,
                                                      const int64_t* expert_start_compact,
                                                      const int64_t* expert_start_tiles, const int64_t* tile_expert,
                                                      const uint8_t* qweight_a, const uint8_t* qweight_b, void* out,
                                                      int32_t out_kind, int64_t compact_rows, int64_t source_rows,
                                                      int64_t in_features, int64_t out_features_a,
                                                      int64_t out_features_b, int64_t num_experts,
                                                      int64_t total_rows, int64_t expert_stride_rows,
                                                      hipStream_t stream) {
  return launch_moe_mmq_wide<GGML_Q8_0>(x_d4s4, compact_to_source, expert_start_compact, expert_start_tiles,
                                        tile_expert, qweight_a, qweight_b, out, out_kind, compact_rows, source_rows,
                                        in_features, out_features_a, out_features_b, num_experts, total_rows,
                                        expert_stride_rows, stream);
}

// The tile map for tiles of any height (hipengine_qwen35_moe_mmq32_tile_map is the 32-row one).
extern "C" int hipengine_gfx950_moe_tile_map(const int64_t* expert_start_compact, int64_t* tile_expert_start,
                                             int64_t* tile_expert, int64_t* total_out, int64_t num_experts,
                                             int64_t tile_capacity, int32_t tile_rows, hipStream_t stream) {
  if (tile_rows != 32 && tile_rows != 64 && tile_rows != 128) return static_cast<int>(hipErrorInvalidValue);
  return launch_tile_map(expert_start_compact, tile_expert_start, tile_expert, total_out, num_experts, tile_capacity,
                         tile_rows, stream);
}

// Router logits in front of the selection; `threads` is accepted and ignored.
#define DEFINE_ROUTER_LOGITS(SYMBOL, HK, WK)                                                                    \
  extern "C" int SYMBOL(const void* hidden, const void* weight, float* logits, int64_t tokens, int64_t hidden_size, \
                        int64_t num_rows, int64_t threads, hipStream_t stream) {                                 \
    return launch_router_logits<HK, WK>(hidden, weight, logits, tokens, hidden_size, num_rows, threads, stream);  \
  }
DEFINE_ROUTER_LOGITS(hipengine_qwen35_router_logits_bf16, KIND_BF16, KIND_BF16)
DEFINE_ROUTER_LOGITS(hipengine_qwen35_router_logits_fp16, KIND_F16, KIND_F16)
DEFINE_ROUTER_LOGITS(hipengine_qwen35_router_logits_bf16_f32w, KIND_BF16, KIND_F32)
DEFINE_ROUTER_LOGITS(hipengine_qwen35_router_logits_fp16_f32w, KIND_F16, KIND_F32)
DEFINE_ROUTER_LOGITS(hipengine_qwen35_router_logits_f32_f32w, KIND_F32, KIND_F32)

extern "C" int hipengine_qwen35_router_select(const float* logits, int64_t* selected, float* routing, int64_t tokens,
                                              int64_t logits_stride, int64_t num_experts, int64_t top_k,
                                              int64_t threads, hipStream_t stream) {
  if (!logits || !selected || !routing || tokens <= 0 || logits_stride <= 0 || num_experts <= 0 || top_k <= 0 ||
      top_k > 16 || top_k > num_experts || num_experts > logits_stride ||
      !(threads == 64 || threads == 128 || threads == 256 || threads == 512) ||
      num_experts > 64 * ROUTER_MAX_PER_LANE) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  const int waves = 4;   // tokens per workgroup; `threads` is accepted and ignored
  const unsigned grid = static_cast<unsigned>((tokens + waves - 1) / waves);
  if (num_experts <= 64 * 4) {
    hipLaunchKernelGGL(router_select_kernel<4>, dim3(grid), dim3(waves * 64), 0, stream, logits, selected, routing,
                       tokens, logits_stride, static_cast<int>(num_experts), static_cast<int>(top_k));
  } else {
    hipLaunchKernelGGL(router_select_kernel<ROUTER_MAX_PER_LANE>, dim3(grid), dim3(waves * 64), 0, stream, logits,
                       selected, routing, tokens, logits_stride, static_cast<int>(num_experts), static_cast<int>(top_k));
  }
  return static_cast<int>(hipGetLastError());
}

int hipengine_gfx950::moe_load() {
  // the Q4_K tile engine holds two copies of a K step's images: more than the 64 KiB a kernel may use unasked
  const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(moe_mmq_kernel<MoeQ4>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize,
                                           static_cast<int>(sizeof(MoeQ4::Smem) + MoeQ4::BM * sizeof(int)));
  if (e != hipSuccess) return static_cast<int>(e);
  hipFuncAttributes attr;
  return static_cast<int>(hipFuncGetAttributes(&attr, reinterpret_cast<const void*>(moe_tile_map_kernel)));
}
