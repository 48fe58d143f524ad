// "Stream" form of the q8_1 decode GEMV for K >= 4096 (nb >= 16 blocks per row),
// batch 1..8: a fixed number of resident waves that walk a contiguous block stream
// with a ring of loads in flight.
//
// Why: a 17408x5120 Q4_K weight is 50 MB, i.e. ~6 us of HBM time.  With one
// short-lived wave per few rows the launch either does not fit the chip in one
// generation (the second generation pays the full load->stage->compute latency
// chain again) or leaves HBM idle while every wave computes.  Here
//   * the grid is sized to the chip (one or two workgroups per CU), all waves are
//     resident from the start and stay until the workgroup's rows are done;
//   * the rows are cut into chunks of R = 16 / gcd(nb, 16) rows (4 rows = 11.5 KB of Q4_K at K = 5120), the
//     fewest whose blocks make whole groups of 16 blocks (2304 B of Q4_K) = one wave-wide load, 4 lanes per
//     block, exactly as in the run form; chunk c belongs to workgroup c % workgroups, and the chunks of a
//     workgroup, in order, are its run;
//   * the waves of the workgroup take the groups of the run round robin (group i*waves + wave in round i).
//     Workgroups advance at about the same pace, so at any time the whole chip reads one window of a few MB
//     that moves through the matrix, every workgroup a different 11.5 KB of it, and the waves are balanced to
//     within one group whatever the rows per workgroup and the wave count.  Measured at 17408x5120 (us per
//     launch, 11 or 12 waves per CU): whole rows per wave 11.4; a contiguous, equal share of blocks per wave
//     12.4 to 16.5 depending on the share's size in bytes; groups round robin within a contiguous share per
//     workgroup 11.7 to 12.0; this form 10.8 to 11.2.
//   * the groups do not divide evenly over the waves; the idle slots are put in round 0,
//     so that the last round, which nothing else hides, is a full one;
//   * D wave loads are kept in flight: after a load's registers are consumed
//     the load D rounds ahead is issued into them, so the stream never drains
//     while the wave computes;
//   * a group touches at most two rows (nb >= 16), so a wave reduces two sums per group
//     with DPP and leaves them in LDS: part[group][0] for the row the group starts in,
//     part[group][1] for the next.  After the workgroup's barrier, thread t adds up the
//     parts of row t in group order (a fixed order: results do not depend on the wave
//     count, on the ring depth or on timing) and stores it: one coalesced store per
//     workgroup and batch row.
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
  int chunk_shift;  // log2 of the rows per chunk R (R * nb is a multiple of 16)
  int base_chunks;  // chunks per workgroup, rounded down (computed on the host: an integer division is ~40
  int extra_chunks; // instructions here); the first extra_chunks workgroups take one more
  int rounds[2];    // rounds of a workgroup with base_chunks / base_chunks + 1 chunks: ceil(groups / waves)
  float inv_nb;     // 1 / (K / 256)
  const uint8_t* w_up;      // FUSE_PAIR: the second matrix (w is the gate), out = silu(gate.x) * (up.x); FUSE_DUAL: the second matrix
  void* out_b;              // FUSE_DUAL: the second matrix's output
  const void* residual;     // FUSE_RESIDUAL: [rows, N] of the output type, added to the projection
  int round_mid;            // FUSE_PAIR: round gate and up to the output type before the SiLU
};

// XK >= 0 fixes the activation kind at compile time (the staging code of the other
// kinds is then not generated: a decode kernel runs its prologue once per launch
// with a cold instruction cache, so prologue code size is launch latency) and
// promises that S groups of 8 values per thread cover K (K/8 <= S * threads/4), so
// the loop over further groups is not generated either (dropping that never-taken
// loop alone took 0.7 us off the 17408x5120 launch); XK < 0 reads the kind from the
// arguments and takes any K.
//
// FUSE selects the epilogue:
//   FUSE_PAIR      the workgroup's run is its rows of the gate matrix followed by the same rows of the
//                  up matrix (groups do not straddle the two); the stored value is silu(gate) * up,
//                  with gate and up rounded to the output type first when round_mid is set
//                  (gguf_q4_k_gemv.hip:652-657);
//   FUSE_RESIDUAL  out = round(projection) + residual in the output type (gguf_q4_k_gemv.hip:1669-1678);
//   FUSE_DUAL      two matrices of one shape as in the pair form, each stored to its own output (gguf_k_gemv.hip:5546-5560).
// The row sums of the three forms are the same floats: the groups of a matrix depend only on the workgroup's rows.
template <int QT, int B, int D, int S, int XK = -1, int FUSE = FUSE_NONE>
__device__ __forceinline__ void gemv_stream_workgroup(const GemvStreamArgs& a, uint8_t* smem, int wg, int grid) {
  using Regs = WeightRegs<GemvTraits<QT>::REGS>;
  constexpr int Q8S = run_q8_stride<QT>();
  constexpr int SUPER = GemvTraits<QT>::SUPER_BYTES;
  constexpr int MATS = (FUSE == FUSE_PAIR || FUSE == FUSE_DUAL) ? 2 : 1;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int q = lane & 3, j = lane >> 2;
  const int nb = a.K / QK_K;

  // the workgroup's chunks wg, wg + workgroups, ...: its run of "virtual" rows and blocks, per matrix
  const int lr = a.chunk_shift;
  const int big = wg < a.extra_chunks ? 1 : 0;
  const int vrows = (a.base_chunks + big) << lr;
  const int total = vrows * nb;                  // blocks of the run: a multiple of 16
  const int ngroups = total >> 4;
  const int rounds = a.rounds[big];
  // round i of this wave is group g_first + i * waves of MATS * ngroups; negative or too large: idle
  const int g_first = wave - (rounds * a.waves - MATS * ngroups);
  // virtual row v is row v + (v >> lr) * gap + (wg << lr) of the matrix
  const int gap = (grid - 1) << lr;
  const int row_off = wg << lr;
  uint8_t* q8 = smem;
  float* rec = reinterpret_cast<float*>(q8 + B * nb * Q8S);
  int* s16 = reinterpret_cast<int*>(rec + B * nb * 16);
  // behind the activation image: part[MATS * ngroups][2][B]
  float* part = reinterpret_cast<float*>(s16 + (QT == GGML_Q6_K ? B * nb * 16 : 0));

  const GemvRunArgs ra{a.x, a.w, a.out, XK >= 0 ? XK : a.x_kind, a.out_kind, a.rows, a.K, a.N, a.waves};
  StageRegs<B, S> sr;
  // The activation loads go first: loads issued after the ring queue behind it (the memory counter retires
  // in order), so a long K wants them all up front: five groups per thread cover K = 17408.  (The weight ring
  // first, which is what the launch waits for, measured slower: 12.5 us against 11.4 at 17408x5120.)
  gemv_run_stage_fetch<QT, B, S>(ra, sr);

  Regs ring[D];
  int ring_row[D], ring_kb[D];                   // this lane's block of the load: virtual row (-1: none) and K block
  // Loads are unconditional (an idle slot reads the block nearest to where it points)
  // so that the number of loads in flight is the same at every step and the
  // waits on the oldest ring slot leave the other D-1 loads outstanding.
  auto issue = [&](int i, Regs& dst, int& dst_row, int& dst_kb) {
    const int g_all = g_first + i * a.waves;                         // over both matrices of the pair form
    int g = g_all;
    const uint8_t* base = a.w;
    if constexpr (MATS == 2) {
      if (g >= ngroups) { g -= ngroups; base = a.w_up; }
    }
    const int blk_raw = g * 16 + j;
    const int blk = min(max(blk_raw, 0), total - 1);
    int v = static_cast<int>((static_cast<float>(blk) + 0.5f) * a.inv_nb);
    if (v * nb > blk) --v;
    if ((v + 1) * nb <= blk) ++v;
    const int kb = blk - v * nb;
    const int row = v + (v >> lr) * gap + row_off;
    const bool live = g_all >= 0 && g_all < MATS * ngroups && row < a.N;     // the last chunk may pass the matrix
    dst_row = live ? v : -1;
    dst_kb = kb;
    gemv_load_block<QT>(base + (static_cast<int64_t>(min(row, a.N - 1)) * nb + kb) * SUPER, q, dst);
  };
#pragma unroll
  for (int c = 0; c < D; ++c) issue(c, ring[c], ring_row[c], ring_kb[c]);

  // the kind-specialised kernels are launched only where the S groups per thread fetched up front cover K
  gemv_run_stage_commit<QT, B, S, (XK >= 0)>(ra, sr, q8, rec, s16);
  __syncthreads();

  for (int i0 = 0; i0 < rounds; i0 += D) {
#pragma unroll
    for (int c = 0; c < D; ++c) {
      const int i = i0 + c;
      const int g_all = g_first + i * a.waves;
      const bool g_live = i < rounds && g_all >= 0 && g_all < MATS * ngroups;   // wave-uniform
      const int row = ring_row[c], kb = ring_kb[c];
      const int row_a = __builtin_amdgcn_readfirstlane(row);         // the row the group starts in
      const BlockScales<QT> s = gemv_block_scales<QT>(ring[c], q);
      float sum_a[B], sum_b[B];
#pragma unroll
      for (int b = 0; b < B; ++b) {
        float term = gemv_run_block_term<QT>(ring[c], s, q, q8 + (b * nb + kb) * Q8S, rec + (b * nb + kb) * 16,
                                             s16 + (b * nb + kb) * 16);
        term = row >= 0 ? term : 0.0f;
        sum_a[b] = (row == row_a) ? term : 0.0f;
        sum_b[b] = (row == row_a) ? 0.0f : term;
      }
      // lane 63 holds the group's last block: does the group reach into a second row?
      const bool two_rows = __builtin_amdgcn_readlane(row, 63) != row_a;
      issue(i + D, ring[c], ring_row[c], ring_kb[c]);
#pragma unroll
      for (int b = 0; b < B; ++b) {
        const float va = wave_sum_to_lane63(sum_a[b]);
        const float vb = two_rows ? wave_sum_to_lane63(sum_b[b]) : 0.0f;
        if (lane == 63 && g_live) {
          part[(g_all * 2 + 0) * B + b] = va;
          part[(g_all * 2 + 1) * B + b] = vb;
        }
      }
    }
  }
  __syncthreads();

  // virtual row t of the workgroup: its blocks [t*nb, (t+1)*nb) lie in groups first..last; the first of them
  // holds the row in slot 0 if the group starts at the row's first block, else in slot 1; the others in slot 0
  for (int t = tid; t < vrows; t += a.waves * 64) {
    const int row = t + (t >> lr) * gap + row_off;
    if (row >= a.N) break;
    const int head = t * nb;
    const int first = head >> 4, last = (head + nb - 1) >> 4;
    const int slot = (first << 4) == head ? 0 : 1;
#pragma unroll
    for (int b = 0; b < B; ++b) {
      if (b >= a.rows) break;
      float v[MATS];
#pragma unroll
      for (int m = 0; m < MATS; ++m) {
        const float* pm = part + m * ngroups * 2 * B;
        float acc = pm[(first * 2 + slot) * B + b];
        for (int g = first + 1; g <= last; ++g) acc += pm[(g * 2) * B + b];
        v[m] = acc;
      }
      const int64_t idx = static_cast<int64_t>(b) * a.N + row;
      if constexpr (FUSE == FUSE_PAIR) {
        float gate = v[0], up = v[MATS - 1];
        if (a.round_mid) { gate = round_to_kind(gate, a.out_kind); up = round_to_kind(up, a.out_kind); }
        const float sig = 1.0f / (1.0f + expf(-gate));
        store_scalar(a.out, idx, gate * sig * up, a.out_kind);
      } else if constexpr (FUSE == FUSE_DUAL) {
        store_scalar(a.out, idx, v[0], a.out_kind);
        store_scalar(a.out_b, idx, v[MATS - 1], a.out_kind);
      } else if constexpr (FUSE == FUSE_RESIDUAL) {
        store_scalar(a.out, idx, round_to_kind(v[0], a.out_kind) + load_scalar(a.residual, idx, a.out_kind), a.out_kind);
      } else {
        store_scalar(a.out, idx, v[0], a.out_kind);
      }
    }
  }
}

}  // namespace hipengine_gfx950
