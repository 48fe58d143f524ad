// "Stream" form of the q8_1 decode GEMV for K >= 4096 (nb >= 16 blocks per row),
// batch 1..8: a fixed number of resident waves, each owning a contiguous range of
// whole rows and walking its block stream with a ring of loads in flight.
//
// Why: a 17408x5120 Q4_K weight is 50 MB, i.e. ~6 us of HBM time.  With one
// short-lived wave per few rows the launch either does not fit the chip in one
// generation (the second generation pays the full load->stage->compute latency
// chain again) or leaves HBM idle while every wave computes.  Here
//   * the grid is sized to the chip (waves_total ~ 8 per CU), all waves are
//     resident from the start and stay until their rows are done;
//   * wave w owns rows [r0, r1) (8 or 9 of them at the C1 shape) = one
//     contiguous run of (r1-r0)*nb blocks, read 16 blocks (2304 B of Q4_K) per
//     wave-wide load, 4 lanes per block, exactly as in the run form;
//   * D wave loads are kept in flight: after a load's registers are consumed
//     the load D steps ahead is issued into them, so the stream never drains
//     while the wave computes;
//   * a wave load touches at most two rows (nb >= 16), so two accumulators per
//     lane suffice: when the stream moves past a row it is reduced across the
//     wave with DPP and stored, and the second accumulator becomes the first.
//
// Activations: whole K, quantized to q8_1 once per workgroup into LDS with the
// padded layout of gguf_gemv_run.hpp.
#pragma once

#include "gguf_gemv_launch.hpp"
#include "gguf_gemv_run.hpp"

namespace hipengine_gfx950 {

struct GemvStreamArgs {
  const void* x;
  const uint8_t* w;
  void* out;
  int x_kind;
  int out_kind;
  int rows;         // batch rows, 1..B
  int K;
  int N;
  int waves;        // waves per workgroup
  int waves_total;  // waves in the whole grid (grid * waves)
  int base_rows;    // N / waves_total (computed on the host: an integer division is ~40 instructions here)
  const uint8_t* w_up;      // FUSE_PAIR: the second matrix (w is the gate); out = silu(gate.x) * (up.x)
  const void* residual;     // FUSE_RESIDUAL: [rows, N] of the output type, added to the projection
  int round_mid;            // FUSE_PAIR: round gate and up to the output type before the SiLU
};

constexpr int STREAM_PAIR_MAX_ROWS = 16;   // rows per wave the pair form can hold back (gate results wait for up)

// XK >= 0 fixes the activation kind at compile time (the staging code of the other
// kinds is then not generated: a decode kernel runs its prologue once per launch
// with a cold instruction cache, so prologue code size is launch latency) and
// promises that S groups of 8 values per thread cover K (K/8 <= S * threads/4), so
// the loop over further groups is not generated either (dropping that never-taken
// loop alone took 0.7 us off the 17408x5120 launch); XK < 0 reads the kind from the
// arguments and takes any K.
//
// FUSE selects the epilogue:
//   FUSE_PAIR      the wave walks its rows of the gate matrix and then the same rows of the up
//                  matrix as one run of 2*nrows rows; gate results wait in LDS (written and read
//                  by lane 63 only) and the stored value is silu(gate) * up, with gate and up
//                  rounded to the output type first when round_mid is set
//                  (gguf_q4_k_gemv.hip:652-657);
//   FUSE_RESIDUAL  out = round(projection) + residual in the output type (gguf_q4_k_gemv.hip:1669-1678).
template <int QT, int B, int D, int S, int XK = -1, int FUSE = FUSE_NONE>
__device__ __forceinline__ void gemv_stream_workgroup(const GemvStreamArgs& a, uint8_t* smem) {
  using Regs = WeightRegs<GemvTraits<QT>::REGS>;
  constexpr int Q8S = run_q8_stride<QT>();
  constexpr int SUPER = GemvTraits<QT>::SUPER_BYTES;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int q = lane & 3, j = lane >> 2;
  const int nb = a.K / QK_K;

  // rows [r0, r0 + nrows) of this wave: N split as evenly as possible
  const int gw = blockIdx.x * a.waves + wave;
  const int base_rows = a.base_rows, extra = a.N - a.base_rows * a.waves_total;
  const int r0 = gw * base_rows + min(gw, extra);
  const int nrows = base_rows + (gw < extra ? 1 : 0);
  const int mat_blocks = nrows * nb;                                   // blocks of this wave in one matrix
  const int run_blocks = FUSE == FUSE_PAIR ? 2 * mat_blocks : mat_blocks;
  const int nloads = (run_blocks + 15) >> 4;
  const uint8_t* wbase = a.w + static_cast<int64_t>(r0) * nb * SUPER;
  const uint8_t* wbase_up = FUSE == FUSE_PAIR ? a.w_up + static_cast<int64_t>(r0) * nb * SUPER : nullptr;

  uint8_t* q8 = smem;
  float* rec = reinterpret_cast<float*>(q8 + B * nb * Q8S);
  int* s16 = reinterpret_cast<int*>(rec + B * nb * 16);
  // pair form: gate results of this wave, [B][STREAM_PAIR_MAX_ROWS], behind the activation image
  float* gate_hold = reinterpret_cast<float*>(s16 + (QT == GGML_Q6_K ? B * nb * 16 : 0)) + wave * B * STREAM_PAIR_MAX_ROWS;

  // Activation loads go first (see gemv_run_stage_fetch), then the weight ring.
  // S activation groups per thread have their loads issued ahead of the weight ring,
  // per batch row.  Loads issued after the ring queue behind it (the memory counter
  // retires in order), so a long K wants them all up front: five cover K = 17408.
  const GemvRunArgs ra{a.x, a.w, a.out, XK >= 0 ? XK : a.x_kind, a.out_kind, a.rows, a.K, a.N, a.waves};
  StageRegs<B, S> sr;
  gemv_run_stage_fetch<QT, B, S>(ra, sr);

  Regs ring[D];
  // Loads are unconditional (indices past the end are clamped to the last block)
  // so that the number of loads in flight is the same at every step and the
  // waits on the oldest ring slot leave the other D-1 loads outstanding.
  const int last_blk = max(run_blocks - 1, 0);
  auto issue = [&](int i, Regs& dst) {
    const int blk = min(i * 16 + j, last_blk);
    if constexpr (FUSE == FUSE_PAIR) {
      const bool up = blk >= mat_blocks;
      gemv_load_block<QT>((up ? wbase_up : wbase) + static_cast<int64_t>(up ? blk - mat_blocks : blk) * SUPER, q, dst);
    } else {
      gemv_load_block<QT>(wbase + static_cast<int64_t>(blk) * SUPER, q, dst);
    }
  };
#pragma unroll
  for (int c = 0; c < D; ++c) issue(c, ring[c]);

  // the kind-specialised kernels are launched only where the S groups per thread fetched up front cover K
  gemv_run_stage_commit<QT, B, S, (XK >= 0)>(ra, sr, q8, rec, s16);
  __syncthreads();

  const int total_rows = FUSE == FUSE_PAIR ? 2 * nrows : nrows;
  float acc_cur[B], acc_next[B];
#pragma unroll
  for (int b = 0; b < B; ++b) { acc_cur[b] = 0.0f; acc_next[b] = 0.0f; }

  // lane state: K block and row (relative to r0) of this lane's block in the current load
  int kb = j, lrow = 0;
  const int step_kb = 16 % nb;                 // nb >= 16: 16 / nb is 0 or 1
  const int step_r = 16 / nb;
  int row_lo = 0, pos_lo = 0;                  // wave-uniform: row of block 16*i and its K block

  auto flush = [&](int row_rel) {
#pragma unroll
    for (int b = 0; b < B; ++b) {
      float v = wave_sum_to_lane63(acc_cur[b]);
      if (lane == 63 && b < a.rows) {
        if constexpr (FUSE == FUSE_PAIR) {
          if (row_rel < nrows) {
            gate_hold[b * STREAM_PAIR_MAX_ROWS + row_rel] = v;
          } else {
            float gate = gate_hold[b * STREAM_PAIR_MAX_ROWS + row_rel - nrows];
            if (a.round_mid) { gate = round_to_kind(gate, a.out_kind); v = round_to_kind(v, a.out_kind); }
            const float sig = 1.0f / (1.0f + expf(-gate));
            store_scalar(a.out, static_cast<int64_t>(b) * a.N + r0 + row_rel - nrows, gate * sig * v, a.out_kind);
          }
        } else if constexpr (FUSE == FUSE_RESIDUAL) {
          const int64_t idx = static_cast<int64_t>(b) * a.N + r0 + row_rel;
          store_scalar(a.out, idx, round_to_kind(v, a.out_kind) + load_scalar(a.residual, idx, a.out_kind), a.out_kind);
        } else {
          store_scalar(a.out, static_cast<int64_t>(b) * a.N + r0 + row_rel, v, a.out_kind);
        }
      }
      acc_cur[b] = acc_next[b];
      acc_next[b] = 0.0f;
    }
  };

  for (int i0 = 0; i0 < nloads; i0 += D) {
#pragma unroll
    for (int c = 0; c < D; ++c) {
      const int i = i0 + c;
      const bool live = i * 16 + j < run_blocks;
      const BlockScales<QT> s = gemv_block_scales<QT>(ring[c], q);
#pragma unroll
      for (int b = 0; b < B; ++b) {
        float term = gemv_run_block_term<QT>(ring[c], s, q, q8 + (b * nb + kb) * Q8S, rec + (b * nb + kb) * 16,
                                             s16 + (b * nb + kb) * 16);
        term = live ? term : 0.0f;
        acc_cur[b] += (lrow == row_lo) ? term : 0.0f;
        acc_next[b] += (lrow == row_lo) ? 0.0f : term;
      }
      issue(i + D, ring[c]);
      // advance the lane to load i+1
      kb += step_kb; lrow += step_r;
      if (kb >= nb) { kb -= nb; lrow += 1; }
      // advance the wave-uniform head; a row is finished once the head passes it
      pos_lo += step_kb;
      int new_lo = row_lo + step_r;
      if (pos_lo >= nb) { pos_lo -= nb; new_lo += 1; }
      if (new_lo > row_lo) {
        if (row_lo < total_rows) flush(row_lo);
        row_lo = new_lo;
      }
    }
  }
  if (row_lo < total_rows) flush(row_lo);
}

}  // namespace hipengine_gfx950
