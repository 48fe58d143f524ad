// "Direct slab" form of the q8_1 decode GEMV, batch 1..8, on the int8 MFMA: the weight blocks go from
// global memory straight into LDS (global_load_lds: no register is held while a load is in flight), so a
// wave keeps a ring of several steps of its weights in flight while it computes, and the stream starts
// before the activations are quantized.
//
// Work decomposition
//   * a workgroup owns a contiguous range of output rows and, when K is split, one of P contiguous parts of
//     K (workgroup index = row group * P + part).  It walks its rows in steps of 16 (the ragged step first:
//     its few rows arrive first and its arithmetic runs while the stream fills);
//   * wave w owns the K blocks w, w + W, ... of the part (at most MAXB of them).  It quantizes only its own
//     K slice of the activations and keeps it in REGISTERS in MFMA operand order;
//   * a unit = (step, all blocks of the wave): 16 rows x nown blocks, fetched by 16-byte chunks, lane l of
//     load k landing at byte 1024 k + 16 l of the unit's LDS slot.  Which global bytes a chunk position
//     holds is the type's choice (DsTraits::chunk_src), so misaligned blocks are realigned and row pitches
//     that would collide on LDS banks are swizzled for free.  A wave has R slots and re-issues a slot as
//     soon as it has read it; loads complete in issue order, so "unit t has landed" is a count of the loads
//     issued after it (s_waitcnt vmcnt);
//   * 16x16 int8 MFMA with the batch as the 16 rows of A and 16 weight rows as the columns of B.  One
//     instruction spans two scale groups (Q4_K / Q8_0: two 32-value sub-blocks of K = 64; Q6_K: the two
//     16-value groups of K = 32); A row m < 8 holds batch row m's values of the first group and zeros in
//     the k range of the second, A row 8 + m the reverse, so lane (n, q) of the result holds, for weight
//     row n, the dots of group q >> 1 with batch rows 4 (q & 1) + v, v = 0..3: every result register of
//     every lane is a wanted dot at batch 8;
//   * the accumulator input of the MFMA is the integer 0x4B400000, so a result reinterpreted as float is
//     12582912 + dot; fma(result, s, -12582912 s) is s * dot exactly for an integer scale s (< 2^24), with
//     no integer conversion; the float scale d of the block is applied once per block;
//   * terms that are a sum over groups of (weight scalar) x (activation scalar) - the Q4_K mins, the
//     -32 * sum(q8) of Q6_K's unsigned 6-bit values - are v_mfma_f32_16x16x4_f32 over the group index;
//   * a group of up to 6 steps keeps its sums in registers; at its end the K slices are added through LDS in
//     wave order (one barrier when the workgroup is a single group).  With K split, the parts' sums go to a
//     partial array in global memory and the workgroup that arrives last adds them in part order: results
//     do not depend on timing.
#pragma once

#include "gguf_gemv_run.hpp"

namespace hipengine_gfx950 {

typedef int ds_v4i __attribute__((ext_vector_type(4)));
typedef uint32_t ds_u32x4 __attribute__((ext_vector_type(4)));
typedef float ds_f4 __attribute__((ext_vector_type(4)));

struct GemvDslabArgs {
  const void* x;
  const uint8_t* w;
  void* out;
  const void* residual;   // null, or [rows, N] of the output type: out = round(projection) + residual
  const void* gate;       // null, or [rows, N] of the output type (may be `out`): out = silu(gate) * round(projection)
  int x_kind;
  int out_kind;
  int rows;        // batch rows, 1..8
  int K;
  int N;
  int waves;       // W
  int ring;        // R: slots (steps in flight) per wave, >= 2
  int base_rows;   // N / row groups; the first N % row groups of them own one row more
  int group;       // steps per group, 1..DS_GROUP
  int red_dedicated;   // 0: every workgroup is a single group (ceil(rows / 16) <= group)
  int ksplit;      // P: parts of K, 1, 2 or 4 (P > 1 needs single-group workgroups)
  int blocks_part; // K blocks per part (the last part takes what is left)
  float* partials;      // P > 1: [P][8][N]
  uint32_t* counters;   // P > 1: one per row group, zero before and after the launch
  int32_t* dots_out;    // verification kernels only: int32 [rows, N, K/32] (Q6_K: K/16), as block_dots writes them
};

constexpr int DS_STEP = 16;                    // rows per step
constexpr int DS_GROUP = 6;                    // steps per group, at most: their sums are kept in registers
constexpr int DS_MAGIC_I = 0x4B400000;         // 12582912.0f: 1.5 * 2^23
constexpr float DS_MAGIC_F = 12582912.0f;
constexpr int DS_SCRATCH = 832;                // staging scratch of a pass: packed [16][32], f32 [16], f32 [16][2], int [16][2]

// Per type: BLK bytes of a block in global memory; the LDS image of (16 rows x one block) = CPR 16-byte
// chunks per row, then DPR dwords per row; chunk_src(p, r) = byte offset inside the block of what chunk
// position p of row r holds; dword_src(i) likewise; REC bytes of LDS records per block kept for the
// whole kernel.
template <int QT>
struct DsTraits;
template <>
struct DsTraits<GGML_Q4_K> {
  static constexpr int BLK = Q4_K_BYTES, CPR = 9, DPR = 0, REC = 0;   // pitch 36 dwords: conflict-free as it lies
  __device__ static __forceinline__ int chunk_src(int p, int) { return 16 * p; }
  __device__ static __forceinline__ int dword_src(int) { return 0; }
};
template <>
struct DsTraits<GGML_Q8_0> {
  // the 8 x 32 values as 16 aligned chunks, position p of row r holding values chunk p ^ r (a pitch of 64 dwords
  // would put the same chunk of all 16 rows on the same banks); the 8 scales as dwords {d, 2 bytes of values}
  static constexpr int BLK = 8 * Q8_0_BYTES, CPR = 16, DPR = 8, REC = 0;
  __device__ static __forceinline__ int chunk_src(int p, int r) {
    const int g = p ^ (r & 15);
    return Q8_0_BYTES * (g >> 1) + 2 + 16 * (g & 1);
  }
  __device__ static __forceinline__ int dword_src(int i) { return Q8_0_BYTES * i; }
};
template <>
struct DsTraits<GGML_Q6_K> {
  // ql (8 chunks), qh (4), scales (1) and the block's last 16 bytes (d in its top half word); rows 8..15 swap
  // neighbouring chunks (pitch 56 dwords: rows r and r + 8 would share banks)
  static constexpr int BLK = Q6_K_BYTES, CPR = 14, DPR = 0, REC = 8 * 8 * 4;   // REC: xd [32-value group][batch row]
  __device__ static __forceinline__ int chunk_src(int p, int r) {
    const int g = p ^ ((r >> 3) & 1);
    return g == 13 ? Q6_K_BYTES - 16 : 16 * g;
  }
  __device__ static __forceinline__ int dword_src(int) { return 0; }
};

template <int QT>
constexpr int ds_image_c() { return DS_STEP * DsTraits<QT>::CPR * 16; }   // chunk section of 16 rows x one block
template <int QT>
constexpr int ds_image_d() { return DS_STEP * DsTraits<QT>::DPR * 4; }    // dword section
template <int QT>
constexpr int ds_image() { return ds_image_c<QT>() + ds_image_d<QT>(); }

// LDS of a workgroup: [partial sums of a group, when the rows are walked in several groups: [W][8][16 * DS_GROUP]
// floats] [the rings: R slots per owned block] [the per-block records]
template <int QT>
constexpr size_t gemv_dslab_lds_bytes(int blocks_part, int waves, int ring, bool red_dedicated) {
  return static_cast<size_t>(red_dedicated ? waves * 512 * DS_GROUP : 0) +
         static_cast<size_t>(ring) * blocks_part * ds_image<QT>() + static_cast<size_t>(blocks_part) * DsTraits<QT>::REC;
}

// Wait until at most n vector-memory operations of this wave are outstanding (n uniform, 0..40).
__device__ __forceinline__ void ds_wait_vm(int n) {
#define DS_WAIT_CASE(N) case N: asm volatile("s_waitcnt vmcnt(" #N ")" ::: "memory"); break;
  switch (n) {
    DS_WAIT_CASE(1) DS_WAIT_CASE(2) DS_WAIT_CASE(3) DS_WAIT_CASE(4) DS_WAIT_CASE(5) DS_WAIT_CASE(6) DS_WAIT_CASE(7)
    DS_WAIT_CASE(8) DS_WAIT_CASE(9) DS_WAIT_CASE(10) DS_WAIT_CASE(11) DS_WAIT_CASE(12) DS_WAIT_CASE(13) DS_WAIT_CASE(14)
    DS_WAIT_CASE(15) DS_WAIT_CASE(16) DS_WAIT_CASE(17) DS_WAIT_CASE(18) DS_WAIT_CASE(19) DS_WAIT_CASE(20) DS_WAIT_CASE(21)
    DS_WAIT_CASE(22) DS_WAIT_CASE(23) DS_WAIT_CASE(24) DS_WAIT_CASE(25) DS_WAIT_CASE(26) DS_WAIT_CASE(27) DS_WAIT_CASE(28)
    DS_WAIT_CASE(29) DS_WAIT_CASE(30) DS_WAIT_CASE(31) DS_WAIT_CASE(32) DS_WAIT_CASE(33) DS_WAIT_CASE(34) DS_WAIT_CASE(35)
    DS_WAIT_CASE(36) DS_WAIT_CASE(37) DS_WAIT_CASE(38) DS_WAIT_CASE(39) DS_WAIT_CASE(40)
    default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
  }
#undef DS_WAIT_CASE
}

// What the dump (verification) instantiation needs to place a dot.
struct DsWhere {
  const GemvDslabArgs* a;
  int kb;            // K block index in the row
  int64_t grow;      // first output row of the step
  int rows_here;     // rows of the step that exist
};

// ---- per type: what a wave keeps in registers for each K block it owns, how the staging fills it, and the
// arithmetic of one block of a unit.  Lane (n = lane & 15, q = lane >> 4) of an MFMA result: weight row n,
// A rows 4q .. 4q+3; p2 = q >> 1 picks which of the instruction's two scale groups, bh = q & 1 the batch half.
//
// Staging: a block is quantized in PASSES passes of 16 teams (4 lanes x 8 values = one 32-value group each);
// team quad = xpar * 8 + batch row takes group group_of(pass, xpar).  After a pass the scratch holds the
// packed values [quad][32], xd [quad] at 512 and two more floats per team at 576 (lane e = 0 writes f0, lane
// e = 2 writes f1; extras() says what they are), and collect() moves what the wave keeps into registers.
template <int QT>
struct DsBlock;

// Q4_K.  MFMA (jp, h), jp = 0, 1 (pairs of 32-byte qs groups), h = 0, 1 (low, high nibbles): lanes q < 2 feed
// the nibbles h of group 2jp, lanes q >= 2 those of group 2jp + 1 - so a lane reads ONE 16-byte chunk
// (chunk 1 + 4jp + q of its row) per pair of instructions and uses both of its nibbles.  The instruction's two
// sub-blocks are 4jp + h (A rows 0..7) and 4jp + 2 + h (A rows 8..15).
// The min term of the block, sum_sb mn_sb * (xd * qsum)_sb, is two v_mfma_f32_16x16x4_f32 (A = xd*qsum by
// batch row and sub-block, B = the 6-bit mins as floats).
template <>
struct DsBlock<GGML_Q4_K> {
  static constexpr int PASSES = 4;     // (jp, h)
  ds_v4i aop[4];                       // A operands, index 2jp + h
  ds_f4 xd[4];                         // xd of batch rows 4bh..4bh+3 for sub-block 4jp + 2p2 + h
  float xs[2];                         // A operands of the min term: (xd*qsum)[batch lane&15][sub-block (lane>>4) + 4i]

  __device__ static __forceinline__ int group_of(int pb, int xpar) { return 4 * (pb >> 1) + 2 * xpar + (pb & 1); }
  __device__ static __forceinline__ void extras(float xd, int part16, int total, float& f0, float& f1) {
    (void)part16;
    f0 = xd * static_cast<float>(total);
    f1 = 0.0f;
  }

  __device__ __forceinline__ void collect(int pb, const uint8_t* sc, int lane, float* rec) {
    (void)rec;
    const int m = lane & 15, c = lane >> 4;
    const ds_v4i got = *reinterpret_cast<const ds_v4i*>(sc + ((c >> 1) * 8 + (m & 7)) * 32 + (c & 1) * 16);
    aop[pb] = (m >> 3) == (c >> 1) ? got : ds_v4i{0, 0, 0, 0};
    xd[pb] = *reinterpret_cast<const ds_f4*>(sc + 512 + ((c >> 1) * 8 + (c & 1) * 4) * 4);
    // min-term operand i = pb >> 1 takes sub-block kq + 4i, kq = lane >> 4: from the pass with h = kq & 1, team half kq >> 1
    const float v = *reinterpret_cast<const float*>(sc + 576 + ((c >> 1) * 8 + (m & 7)) * 8);
    if ((pb & 1) == 0) xs[pb >> 1] = 0.0f;
    const bool mine = (c & 1) == (pb & 1) && m < 8;
    xs[pb >> 1] = mine ? v : xs[pb >> 1];
  }

  template <bool VERIFY>
  __device__ __forceinline__ void compute(const uint8_t* img, const uint8_t* imgd, const float* rec, int lane, float (&acc)[4],
                                          const DsWhere& wh) const {
    (void)imgd; (void)rec;
    const int n = lane & 15, q = lane >> 4, p2 = q >> 1, bh = q & 1;
    const uint8_t* wl = img + n * Q4_K_BYTES;
    const ds_u32x4 hd = *reinterpret_cast<const ds_u32x4*>(wl);
    const ds_u32x4 qs0 = *reinterpret_cast<const ds_u32x4*>(wl + 16 + 16 * q);
    const ds_u32x4 qs1 = *reinterpret_cast<const ds_u32x4*>(wl + 80 + 16 * q);
    const Q4KScales u = q4k_unpack_scales(hd.y, hd.z, hd.w);
    const float d = f16_bits_to_float(hd.x & 0xFFFFu);
    const float ndmin = -f16_bits_to_float(hd.x >> 16);
    // this lane's sub-blocks 4jp + 2p2 + h: bytes 2p2 + h of the low (jp = 0) and high (jp = 1) scale words
    const uint32_t scw[2] = {u.sc_lo >> (16 * p2), u.sc_hi >> (16 * p2)};
    // min term: B operand = min of sub-block q + 4i of row n
    ds_f4 mt = ds_f4{0.0f, 0.0f, 0.0f, 0.0f};
    mt = __builtin_amdgcn_mfma_f32_16x16x4f32(xs[0], static_cast<float>((u.mn_lo >> (8 * q)) & 0xFFu), mt, 0, 0, 0);
    mt = __builtin_amdgcn_mfma_f32_16x16x4f32(xs[1], static_cast<float>((u.mn_hi >> (8 * q)) & 0xFFu), mt, 0, 0, 0);
    const ds_v4i magic = ds_v4i{DS_MAGIC_I, DS_MAGIC_I, DS_MAGIC_I, DS_MAGIC_I};
    float part[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int jp = 0; jp < 2; ++jp) {
      const ds_u32x4 qs = jp == 0 ? qs0 : qs1;
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        ds_v4i wop;
#pragma unroll
        for (int c = 0; c < 4; ++c) wop[c] = static_cast<int>(h == 0 ? q4k_low(qs[c]) : q4k_high(qs[c]));
        const ds_v4i r = __builtin_amdgcn_mfma_i32_16x16x64_i8(aop[2 * jp + h], wop, magic, 0, 0, 0);
        const float scf = static_cast<float>((scw[jp] >> (8 * h)) & 0xFFu);
        const float swm = -DS_MAGIC_F * scf;
        if constexpr (VERIFY) {
          const int sb = 4 * jp + 2 * p2 + h;
#pragma unroll
          for (int v = 0; v < 4; ++v) {
            const int m = 4 * bh + v;
            if (m < wh.a->rows && n < wh.rows_here)
              wh.a->dots_out[(static_cast<int64_t>(m) * wh.a->N + wh.grow + n) * (wh.a->K / 32) + wh.kb * 8 + sb] = r[v] - DS_MAGIC_I;
          }
        }
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const int rv = r[v];   // by value: a bit cast of the vector element itself reads element 0
          const float tv = __builtin_fmaf(bits_to_float(static_cast<uint32_t>(rv)), scf, swm);   // sc * dot, exact
          part[v] = __builtin_fmaf(xd[2 * jp + h][v], tv, part[v]);
        }
      }
    }
#pragma unroll
    for (int v = 0; v < 4; ++v) acc[v] = __builtin_fmaf(d, part[v], __builtin_fmaf(ndmin, mt[v], acc[v]));
  }
};

// Q8_0.  MFMA i = 0..3 takes the 32-value blocks 2i (A rows 0..7) and 2i + 1 (A rows 8..15): lane (n, q) reads
// values chunk 4i + q of its row (at position (4i + q) ^ n) and the scale dword of block 2i + (q >> 1).
template <>
struct DsBlock<GGML_Q8_0> {
  static constexpr int PASSES = 4;
  ds_v4i aop[4];
  ds_f4 xd[4];

  __device__ static __forceinline__ int group_of(int pb, int xpar) { return 2 * pb + xpar; }
  __device__ static __forceinline__ void extras(float, int, int, float& f0, float& f1) { f0 = 0.0f; f1 = 0.0f; }

  __device__ __forceinline__ void collect(int pb, const uint8_t* sc, int lane, float* rec) {
    (void)rec;
    const int m = lane & 15, c = lane >> 4;
    const ds_v4i got = *reinterpret_cast<const ds_v4i*>(sc + ((c >> 1) * 8 + (m & 7)) * 32 + (c & 1) * 16);
    aop[pb] = (m >> 3) == (c >> 1) ? got : ds_v4i{0, 0, 0, 0};
    xd[pb] = *reinterpret_cast<const ds_f4*>(sc + 512 + ((c >> 1) * 8 + (c & 1) * 4) * 4);
  }

  template <bool VERIFY>
  __device__ __forceinline__ void compute(const uint8_t* img, const uint8_t* imgd, const float* rec, int lane, float (&acc)[4],
                                          const DsWhere& wh) const {
    (void)rec;
    const int n = lane & 15, q = lane >> 4, p2 = q >> 1, bh = q & 1;
    const uint8_t* wl = img + n * 256;
    const ds_u32x4 dlo = *reinterpret_cast<const ds_u32x4*>(imgd + n * 32 + 16 * 0);
    const ds_u32x4 dhi = *reinterpret_cast<const ds_u32x4*>(imgd + n * 32 + 16);
    const ds_v4i magic = ds_v4i{DS_MAGIC_I, DS_MAGIC_I, DS_MAGIC_I, DS_MAGIC_I};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const ds_v4i wop = *reinterpret_cast<const ds_v4i*>(wl + 16 * ((4 * i + q) ^ n));
      const ds_v4i r = __builtin_amdgcn_mfma_i32_16x16x64_i8(aop[i], wop, magic, 0, 0, 0);
      // scale of block 2i + p2: dword 2i + p2 of the row's eight
      const uint32_t e0 = i < 2 ? dlo[2 * (i & 1)] : dhi[2 * (i & 1)], e1 = i < 2 ? dlo[2 * (i & 1) + 1] : dhi[2 * (i & 1) + 1];
      const float dw = f16_bits_to_float((p2 ? e1 : e0) & 0xFFFFu);
      const float dwm = -DS_MAGIC_F * dw;     // 12582912 * dw is exact: dw has 11 significant bits
      if constexpr (VERIFY) {
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const int m = 4 * bh + v;
          if (m < wh.a->rows && n < wh.rows_here)
            wh.a->dots_out[(static_cast<int64_t>(m) * wh.a->N + wh.grow + n) * (wh.a->K / 32) + wh.kb * 8 + 2 * i + p2] = r[v] - DS_MAGIC_I;
        }
      }
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int rv = r[v];
        const float tv = __builtin_fmaf(bits_to_float(static_cast<uint32_t>(rv)), dw, dwm);   // dw * dot, one rounding
        acc[v] = __builtin_fmaf(xd[i][v], tv, acc[v]);
      }
    }
  }
};

// Q6_K.  v_mfma_i32_16x16x32_i8 (h, qt): the 32 values qt of half h - 16-value groups 8h + 2qt (A rows 0..7,
// k 0..15) and 8h + 2qt + 1 (A rows 8..15, k 16..31), which have their own int8 scales.  Lane (n, q) takes
// values 8q .. 8q+7 of each of the half's four 32-value runs from 8 bytes of ql[64h + 8q], ql[64h + 32 + 8q]
// and qh[32h + 8q]: three reads feed four instructions.  B holds the unsigned 6-bit values; the -32 * sum(q8)
// that makes the dot signed is, per block, sum over 16-value groups of sc_g * (-32 * xd * qsum16_g): four
// v_mfma_f32_16x16x4_f32 (the verification kernel subtracts per dot instead).
template <>
struct DsBlock<GGML_Q6_K> {
  static constexpr int PASSES = 4;     // pass pb: 32-value groups 2pb and 2pb + 1
  long aop[8];                         // A operands by 32-value group 4h + qt
  ds_v4i vq[8];                        // verification only: qsum16 of batch rows 4bh..4bh+3, 16-value group 2 (4h + qt) + p2
  float cs[4];                         // A operands of the correction: (-32 xd qsum16)[batch lane&15][group (lane>>4) + 4i]

  __device__ static __forceinline__ int group_of(int pb, int xpar) { return 2 * pb + xpar; }
  __device__ static __forceinline__ void extras(float xd, int part16, int, float& f0, float& f1) {
    // lanes e = 0, 1 of a team hold the sum of its first 16 values, lanes e = 2, 3 that of the second 16
    f0 = -32.0f * xd * static_cast<float>(part16);
    f1 = f0;
  }

  __device__ __forceinline__ void collect(int pb, const uint8_t* sc, int lane, float* rec) {
    const int m = lane & 15, c = lane >> 4;
    const bool nonzero = (m >> 3) == (c >> 1);
#pragma unroll
    for (int g = 0; g < 2; ++g) {
      const uint2 got = *reinterpret_cast<const uint2*>(sc + (g * 8 + (m & 7)) * 32 + 8 * c);
      const uint64_t v = static_cast<uint64_t>(got.x) | (static_cast<uint64_t>(got.y) << 32);
      aop[2 * pb + g] = nonzero ? static_cast<long>(v) : 0l;
    }
    // xd of the pass's two groups, all batch rows, to the records: lanes 0..15 <- team quad = lane
    if (lane < 16) rec[(2 * pb + (lane >> 3)) * 8 + (lane & 7)] = *reinterpret_cast<const float*>(sc + 512 + lane * 4);
    // correction operand i = pb: 16-value group c + 4 pb = half c & 1 of 32-value group 2 pb + (c >> 1)
    const float v = *reinterpret_cast<const float*>(sc + 576 + ((c >> 1) * 8 + (m & 7)) * 8 + (c & 1) * 4);
    cs[pb] = m < 8 ? v : 0.0f;
#pragma unroll
    for (int g = 0; g < 2; ++g)
#pragma unroll
      for (int vv = 0; vv < 4; ++vv)
        vq[2 * pb + g][vv] = *reinterpret_cast<const int*>(sc + 704 + ((g * 8 + 4 * (c & 1) + vv) * 2 + (c >> 1)) * 4);
  }

  template <bool VERIFY>
  __device__ __forceinline__ void compute(const uint8_t* img, const uint8_t* imgd, const float* rec, int lane, float (&acc)[4],
                                          const DsWhere& wh) const {
    (void)imgd;
    const int n = lane & 15, q = lane >> 4, p2 = q >> 1, bh = q & 1;
    const uint8_t* wl = img + n * 224;
    const int sw = (n >> 3) & 1;                                   // rows 8..15: neighbouring chunks swapped
    auto at = [&](int byte) { return wl + (((byte >> 4) ^ sw) << 4) + (byte & 15); };
    const ds_u32x4 scw = *reinterpret_cast<const ds_u32x4*>(at(192));
    const float d = f16_bits_to_float(*reinterpret_cast<const uint32_t*>(at(208 + 12)) >> 16);
    // correction: B operand = scale of 16-value group q + 4i of row n
    ds_f4 ct = ds_f4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int s8 = static_cast<int>(scw[i] << (24 - 8 * q)) >> 24;
      ct = __builtin_amdgcn_mfma_f32_16x16x4f32(cs[i], static_cast<float>(s8), ct, 0, 0, 0);
    }
    const ds_v4i magic = ds_v4i{DS_MAGIC_I, DS_MAGIC_I, DS_MAGIC_I, DS_MAGIC_I};
    float part[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const uint2 qla = *reinterpret_cast<const uint2*>(at(64 * h + 8 * q));
      const uint2 qlb = *reinterpret_cast<const uint2*>(at(64 * h + 32 + 8 * q));
      const uint2 qhh = *reinterpret_cast<const uint2*>(at(128 + 32 * h + 8 * q));
      const Q6KQuad ux = q6k_unpack(qla.x, qlb.x, qhh.x), uy = q6k_unpack(qla.y, qlb.y, qhh.y);
#pragma unroll
      for (int qt = 0; qt < 4; ++qt) {
        const uint32_t wx = qt == 0 ? ux.g0 : qt == 1 ? ux.g1 : qt == 2 ? ux.g2 : ux.g3;
        const uint32_t wy = qt == 0 ? uy.g0 : qt == 1 ? uy.g1 : qt == 2 ? uy.g2 : uy.g3;
        const long wop = static_cast<long>(static_cast<uint64_t>(wx) | (static_cast<uint64_t>(wy) << 32));
        const ds_v4i r = __builtin_amdgcn_mfma_i32_16x16x32_i8(aop[4 * h + qt], wop, magic, 0, 0, 0);
        // int8 scale of 16-value group 8h + 2qt + p2: byte 2 (qt & 1) + p2 of word 2h + (qt >> 1)
        const int s8 = static_cast<int>(scw[2 * h + (qt >> 1)] << (24 - 16 * (qt & 1) - 8 * p2)) >> 24;
        const float scf = static_cast<float>(s8);
        const float swm = -DS_MAGIC_F * scf;
        const ds_f4 xd4 = *reinterpret_cast<const ds_f4*>(rec + (4 * h + qt) * 8 + 4 * bh);
        if constexpr (VERIFY) {
          // signed dot = unsigned dot - 32 * qsum16
          const int g16 = 8 * h + 2 * qt + p2;
#pragma unroll
          for (int v = 0; v < 4; ++v) {
            const int m = 4 * bh + v;
            if (m < wh.a->rows && n < wh.rows_here)
              wh.a->dots_out[(static_cast<int64_t>(m) * wh.a->N + wh.grow + n) * (wh.a->K / 16) + wh.kb * 16 + g16] =
                  r[v] - DS_MAGIC_I - 32 * vq[4 * h + qt][v];
          }
        }
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const int rv = r[v];
          const float tv = __builtin_fmaf(bits_to_float(static_cast<uint32_t>(rv)), scf, swm);   // sc * dot_u, exact
          part[v] = __builtin_fmaf(xd4[v], tv, part[v]);
        }
      }
    }
#pragma unroll
    for (int v = 0; v < 4; ++v) acc[v] = __builtin_fmaf(d, part[v] + ct[v], acc[v]);
  }
};

// XK fixes the activation kind at compile time (the staging code of the other kinds is not generated).
template <int QT, int MAXB, int XK, bool VERIFY = false>
__device__ __forceinline__ void gemv_dslab_workgroup(const GemvDslabArgs& a, uint8_t* smem) {
  using T = DsTraits<QT>;
  using Blk = DsBlock<QT>;
  constexpr int BLK = T::BLK, CPR = T::CPR, DPR = T::DPR;
  constexpr int IMG_C = ds_image_c<QT>(), IMG_D = ds_image_d<QT>(), IMG = IMG_C + IMG_D;
  constexpr int LC_MAX = (MAXB * DS_STEP * CPR + 63) / 64;         // 16-byte loads per unit, at most
  constexpr int LD_MAX = (MAXB * DS_STEP * DPR + 63) / 64;         // 4-byte loads per unit, at most

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int nb = a.K / QK_K;
  const int W = a.waves, R = a.ring, P = a.ksplit;
  const int row_bytes = nb * BLK;

  // rows and K part of this workgroup
  const int wg = static_cast<int>(blockIdx.x), n_rg = static_cast<int>(gridDim.x) / P;
  const int rg = wg / P, part = wg - rg * P;
  const int extra = a.N - a.base_rows * n_rg;
  const int r_begin = rg * a.base_rows + min(rg, extra);
  const int nrows = a.base_rows + (rg < extra ? 1 : 0);
  if (nrows <= 0) return;   // uniform over the workgroup
  const int steps = (nrows + DS_STEP - 1) / DS_STEP;
  const int first = nrows - DS_STEP * (steps - 1);                 // rows of step 0 (the ragged one), 1..16
  auto step_row = [&](int t) { return t == 0 ? 0 : first + DS_STEP * (t - 1); };
  auto step_rows = [&](int t) { return t == 0 ? first : DS_STEP; };
  const int kb0 = part * a.blocks_part;                            // first K block of the part
  const int nbp = min(a.blocks_part, nb - kb0);                    // its blocks

  // blocks of this wave: kb0 + w, kb0 + w + W, ...; `before` = blocks owned by the waves in front of it
  auto owned = [&](int w_) { return max(0, (nbp - w_ + W - 1) / W); };
  const int nown = owned(wave);                                    // 0..MAXB
  int before = 0;
  for (int i = 0; i < wave; ++i) before += owned(i);

  uint8_t* ring_all = smem + (a.red_dedicated ? W * 512 * DS_GROUP : 0);
  uint8_t* ring = ring_all + before * R * IMG;                     // this wave's R slots of nown * IMG bytes
  float* rec_all = reinterpret_cast<float*>(ring_all + a.blocks_part * R * IMG);
  const int slot_bytes = nown * IMG;
  const uint32_t ring_lds = lds_address(ring);

  // ---- load plan.  16-byte chunk ci = 64 k + lane of the unit's chunk section [block][row][position], then
  // dword di = 64 k + lane of its dword section [block][row][index].  vfull = the lane's offset from the first
  // byte of the step's first row when all 16 rows exist; rows4 = the rows of the lane's loads, 4 bits each.
  const int unit_chunks = nown * DS_STEP * CPR, unit_dwords = nown * DS_STEP * DPR;
  const int LC = (unit_chunks + 63) >> 6, LD = (unit_dwords + 63) >> 6, L = LC + LD;
  uint32_t vfull[LC_MAX + LD_MAX];
  uint64_t rows4 = 0;
#pragma unroll
  for (int k = 0; k < LC_MAX; ++k) {
    const int ci = max(0, min(64 * k + lane, unit_chunks - 1));
    const int s = ci / (DS_STEP * CPR), rem = ci - s * (DS_STEP * CPR);
    const int row = rem / CPR, p = rem - row * CPR;
    vfull[k] = static_cast<uint32_t>(row * row_bytes + (kb0 + wave + s * W) * BLK + T::chunk_src(p, row));
    rows4 |= static_cast<uint64_t>(row) << (4 * k);
  }
#pragma unroll
  for (int k = 0; k < LD_MAX; ++k) {
    const int di = max(0, min(64 * k + lane, unit_dwords - 1));
    const int s = di / (DS_STEP * (DPR ? DPR : 1)), rem = di - s * (DS_STEP * DPR);
    const int row = rem / (DPR ? DPR : 1), i = rem - row * DPR;
    vfull[LC_MAX + k] = static_cast<uint32_t>(row * row_bytes + (kb0 + wave + s * W) * BLK + T::dword_src(i));
    rows4 |= static_cast<uint64_t>(row) << (4 * (LC_MAX + k));
  }
  auto issue = [&](int t) {
    const uint8_t* base = a.w + static_cast<int64_t>(r_begin + step_row(t)) * row_bytes;
    const int last = step_rows(t) - 1;
    const uint32_t slot = ring_lds + static_cast<uint32_t>((t % R) * slot_bytes);
    // rows past the step's last are clamped to it (their results are dropped): every load is issued, so the
    // count that the waits rely on does not depend on the step
    auto offset = [&](int k) {
      const int row = static_cast<int>(rows4 >> (4 * k)) & 15;
      return last == DS_STEP - 1 ? vfull[k] : vfull[k] - static_cast<uint32_t>(__mul24(max(row - last, 0), row_bytes));
    };
#pragma unroll
    for (int k = 0; k < LC_MAX; ++k) {
      if (k < LC) {
        if (64 * k + lane < unit_chunks) lds_dma16(base, offset(k), slot + 1024u * k);
      }
    }
#pragma unroll
    for (int k = 0; k < LD_MAX; ++k) {
      if (k < LD) {
        if (64 * k + lane < unit_dwords) lds_dma4(base, offset(LC_MAX + k), slot + static_cast<uint32_t>(nown * IMG_C) + 256u * k);
      }
    }
  };

  // ---- activation loads of this wave's K slice: 4 lanes per 32-value group, 8 values per lane, 16 groups per
  // pass.  Pass p = (owned block p / PB, pass pb of the block).
  constexpr int PB = Blk::PASSES;
  constexpr int PASSES = MAXB * PB;
  const int quad = lane >> 2, e = lane & 3;
  const int xb = quad & 7, xpar = quad >> 3;
  const int xrow = min(xb, a.rows - 1);                            // clamped: rows past the batch are zeroed below
  uint32_t raw[PASSES][8];
#pragma unroll
  for (int p = 0; p < PASSES; ++p) {
#pragma unroll
    for (int i = 0; i < 8; ++i) raw[p][i] = 0u;
    if (p / PB < nown) {
      const int j = (kb0 + wave + (p / PB) * W) * 8 + Blk::group_of(p % PB, xpar);   // 32-value group of the row
      if (XK == KIND_F32) {
        const uint4* src = reinterpret_cast<const uint4*>(static_cast<const float*>(a.x) + static_cast<int64_t>(xrow) * a.K + j * 32 + e * 8);
        const uint4 lo = src[0], hi = src[1];
        raw[p][0] = lo.x; raw[p][1] = lo.y; raw[p][2] = lo.z; raw[p][3] = lo.w;
        raw[p][4] = hi.x; raw[p][5] = hi.y; raw[p][6] = hi.z; raw[p][7] = hi.w;
      } else if (XK == KIND_Q8_1) {
        const uint8_t* blk = static_cast<const uint8_t*>(a.x) + (static_cast<int64_t>(xrow) * (a.K / 32) + j) * Q8_1_BYTES;
        raw[p][0] = *reinterpret_cast<const uint32_t*>(blk + 4 + 8 * e);
        raw[p][1] = *reinterpret_cast<const uint32_t*>(blk + 8 + 8 * e);
        raw[p][2] = *reinterpret_cast<const uint32_t*>(blk);
      } else {
        const uint4 h = *reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(a.x) + static_cast<int64_t>(xrow) * a.K + j * 32 + e * 8);
        raw[p][0] = h.x; raw[p][1] = h.y; raw[p][2] = h.z; raw[p][3] = h.w;
      }
    }
  }
  // All of them have to be here before the first weight load is issued: the compiler's waits for them count
  // loads in issue order and would otherwise wait for the weight stream as well.
  constexpr int RAW_USED = XK == KIND_F32 ? 8 : XK == KIND_Q8_1 ? 3 : 4;
#pragma unroll
  for (int p = 0; p < PASSES; ++p)
#pragma unroll
    for (int i = 0; i < RAW_USED; ++i) asm volatile("" : "+v"(raw[p][i]));

  // the stream starts: every slot but the last, which the staging below uses as its scratch
  const int ahead = min(R - 1, steps);
  if (nown > 0) {
    for (int t = 0; t < ahead; ++t) issue(t);
  }

  // ---- quantize the slice; operands to registers through the scratch (two buffers, by pass parity)
  uint8_t* scratch = ring + (R - 1) * slot_bytes;
  Blk blk[MAXB];
#pragma unroll
  for (int p = 0; p < PASSES; ++p) {
    if (p / PB < nown) {
      uint32_t packed[2];
      float xd;
      q8_quantize8(XK, raw[p], true, packed, xd);
      const bool used = xb < a.rows;
      packed[0] = used ? packed[0] : 0u;
      packed[1] = used ? packed[1] : 0u;
      xd = used ? xd : 0.0f;
      int part16 = dot4(0x01010101u, packed[1], dot4(0x01010101u, packed[0], 0));
      part16 += dpp_i<DPP_QUAD_XOR1>(part16);
      const int total = part16 + dpp_i<DPP_QUAD_XOR2>(part16);
      float f0, f1;
      Blk::extras(xd, part16, total, f0, f1);
      uint8_t* sc = scratch + (p & 1) * DS_SCRATCH;
      *reinterpret_cast<uint2*>(sc + quad * 32 + e * 8) = make_uint2(packed[0], packed[1]);
      if (e == 0) {
        reinterpret_cast<float*>(sc + 512)[quad] = xd;
        reinterpret_cast<float*>(sc + 576)[2 * quad] = f0;
      }
      if (e == 2) reinterpret_cast<float*>(sc + 576)[2 * quad + 1] = f1;
      if (e == 0 || e == 2) reinterpret_cast<int*>(sc + 704)[2 * quad + (e >> 1)] = part16;   // sums of the two 16-value halves
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      blk[p / PB].collect(p % PB, sc, lane, rec_all + (before + p / PB) * (T::REC / 4));
    }
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");               // the scratch has been read: the slot may be loaded
  if (nown > 0 && R - 1 < steps) issue(R - 1);

  // ---- main loop: groups of at most `group` steps; a step's sums stay in four registers until the group ends
  const int n = lane & 15, q = lane >> 4;
  const int G = a.group;
  // partial sums of a group, [batch row][16 * step of the group + row]: in the wave's own ring when the whole
  // workgroup is one group (the stream has ended by then), else in an array of their own in front of the rings
  float* my_red = reinterpret_cast<float*>(a.red_dedicated ? smem + wave * (512 * DS_GROUP) : ring);
  for (int t0 = 0; t0 < steps; t0 += G) {
    const int gsteps = min(G, steps - t0);
    float done[DS_GROUP][4];
#pragma unroll
    for (int u = 0; u < DS_GROUP; ++u)
#pragma unroll
      for (int v = 0; v < 4; ++v) done[u][v] = 0.0f;
    if (nown > 0) {
#pragma unroll 1
      for (int tt = 0; tt < gsteps; ++tt) {
        const int t = t0 + tt;
        // units t+1 .. are behind unit t in the queue: wait until only they are outstanding
        const int later = min(t + R, steps) - t - 1;
        ds_wait_vm(later * L);
        const uint8_t* slot = ring + (t % R) * slot_bytes;
        float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        DsWhere wh{&a, 0, r_begin + step_row(t), step_rows(t)};
#pragma unroll
        for (int s = 0; s < MAXB; ++s) {
          if (s < nown) {
            wh.kb = kb0 + wave + s * W;
            blk[s].template compute<VERIFY>(slot + s * IMG_C, slot + nown * IMG_C + s * IMG_D,
                                            rec_all + (before + s) * (T::REC / 4), lane, acc, wh);
          }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");         // the slot has been read
        if (t + R < steps) issue(t + R);
#pragma unroll
        for (int u = 0; u < DS_GROUP; ++u)
#pragma unroll
          for (int v = 0; v < 4; ++v) done[u][v] = (u == tt) ? acc[v] : done[u][v];
      }
      // the two scale groups of a (row, batch row) sit 32 lanes apart
#pragma unroll
      for (int u = 0; u < DS_GROUP; ++u) {
        if (u < gsteps) {
#pragma unroll
          for (int v = 0; v < 4; ++v) {
            const float sum = done[u][v] + __shfl_xor(done[u][v], 32);
            if (lane < 32) my_red[(4 * q + v) * (16 * DS_GROUP) + 16 * u + n] = sum;
          }
        }
      }
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    // K slices added in wave order: thread -> (batch row, step of the group, row of the step)
    const int nwork = min(W, nbp);                                 // waves that own blocks
    auto for_outputs = [&](auto&& body) {
      for (int idx = tid; idx < a.rows * 16 * gsteps; idx += W * 64) {
        const int m = idx / (16 * gsteps), j = idx - m * 16 * gsteps;
        const int t = t0 + (j >> 4), rl = j & 15;
        if (rl < step_rows(t)) body(m, j, static_cast<int64_t>(m) * a.N + r_begin + step_row(t) + rl);
      }
    };
    auto finish = [&](float v, int64_t oi) {
      if (a.residual) v = round_to_kind(v, a.out_kind) + load_scalar(a.residual, oi, a.out_kind);
      if (a.gate) {   // the up half of a gate/up pair: the gate projection is already stored, rounded
        const float gt = load_scalar(a.gate, oi, a.out_kind);
        const float sig = 1.0f / (1.0f + expf(-gt));
        v = gt * sig * round_to_kind(v, a.out_kind);
      }
      store_scalar(a.out, oi, v, a.out_kind);
    };
    auto slice_sum = [&](int m, int j) {
      float v = 0.0f;
      int off = 0;   // of wave s's partial sums
      for (int s = 0; s < nwork; ++s) {
        const float* src = reinterpret_cast<const float*>(a.red_dedicated ? smem + s * (512 * DS_GROUP) : ring_all + off);
        v += src[m * (16 * DS_GROUP) + j];
        off += owned(s) * R * IMG;
      }
      return v;
    };
    if (P == 1) {
      for_outputs([&](int m, int j, int64_t oi) { finish(slice_sum(m, j), oi); });
    } else {
      // this part's sums to the partial array; the workgroup of the row group that arrives last adds the
      // parts in order.  The partial sums travel as device-scope accesses (written through to, and read from,
      // the level all workgroups share) and the arrival counter is incremented after the stores have completed:
      // no cache-wide write-back or invalidation is needed.
      for_outputs([&](int m, int j, int64_t oi) {
        __hip_atomic_store(a.partials + static_cast<int64_t>(part) * 8 * a.N + oi, slice_sum(m, j), __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
      });
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
      uint32_t* flag = reinterpret_cast<uint32_t*>(smem);
      if (tid == 0) *flag = __hip_atomic_fetch_add(a.counters + rg, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __syncthreads();
      const bool last = *flag == static_cast<uint32_t>(P - 1);
      if (last) {
        for_outputs([&](int, int, int64_t oi) {
          float v = 0.0f;
          for (int p = 0; p < P; ++p)
            v += __hip_atomic_load(a.partials + static_cast<int64_t>(p) * 8 * a.N + oi, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          finish(v, oi);
        });
        if (tid == 0) __hip_atomic_store(a.counters + rg, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    if (t0 + G < steps) asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");   // the sums have been read
  }
}

}  // namespace hipengine_gfx950
