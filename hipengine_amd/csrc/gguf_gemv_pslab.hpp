// "Phased slab" form of the q8_1 decode GEMV for Q5_K, Q6_K and Q8_0 weights (and Q4_K rows
// too long for the slab form), batch 3..8, on the int8 MFMA, for any K that is a multiple of 512.
//
// Why: the v_dot4 forms do the weight unpacking once but the dot products once per
// batch row, so at batch 8 they are bound by VALU issue (a 5120x17408 Q6_K matrix takes
// four times as long as at batch 1).  On the MFMA the batch rides along: the VALU unpacks
// each weight once and applies scales to 4 results per lane and sub-block.
//
// Work decomposition
//   * a workgroup owns a contiguous range of output rows and walks it in groups of up
//     to 96 rows = 3 steps of 32;
//   * its W waves split K by 256-value blocks: wave w owns blocks
//     (p*bpw + s)*W + w, s < bpw, of every phase p.  With one phase (W*bpw >= K/256) the
//     wave quantizes its K slice of the activations once into wave-private LDS and keeps
//     it for all row groups; with several phases a workgroup has a single row group and
//     the wave re-quantizes its bpw blocks at the start of each phase (the whole
//     quantized activation of K = 17408 at batch 8 does not fit the LDS);
//   * a unit of work is (owned block j, step t): the wave loads the 32 x BLK bytes with
//     16-byte buffer loads that are contiguous along each row, copies them to
//     wave-private LDS and reads them back in MFMA operand order (lane (n, g) = row n,
//     k half g).  The loads of the next unit are issued before the current one is
//     computed.  Q6_K blocks are 210 bytes, so a block starts 0 or 2 bytes past a
//     4-byte boundary: the buffer loads start at the block (2-byte aligned loads run at
//     full rate) so that its LDS image, and every LDS read of it, is 16-byte aligned;
//   * Q6_K: v_mfma_i32_32x32x16_i8 per 16-value group with B = the unsigned 6-bit values;
//     adding -32 * sum(q8 of the group) of the batch row gives the signed dot of
//     gguf_k_gemv.hip:233-246 (a shared all-zero accumulator input: a per-instruction
//     one costs a dozen register moves each); per 32 values
//     acc += xd * float(sc0*dot0 + sc1*dot1), and d once per block;
//     Q8_0: v_mfma_i32_32x32x32_i8 per 34-byte block, acc += xd * (d * float(dot))
//     (gguf_q8_0_dp4a_gemv.hip:122-129);
//   * K slices are summed through LDS in wave order; two workgroup barriers per row group.
#pragma once

#include "gguf_gemv_run.hpp"

namespace hipengine_gfx950 {

typedef int ps_v4i __attribute__((ext_vector_type(4)));
typedef int ps_v16i __attribute__((ext_vector_type(16)));
typedef uint32_t ps_u32x4 __attribute__((ext_vector_type(4)));
typedef float ps_f4 __attribute__((ext_vector_type(4)));

struct GemvPslabArgs {
  const void* x;
  const uint8_t* w;
  void* out;
  const void* residual;   // null, or [rows, N] of the output type: out = round(projection) + residual
  const void* gate;       // null, or [rows, N] of the output type (may be `out` itself): out = silu(gate) * round(projection)
  int x_kind;
  int out_kind;
  int rows;        // batch rows, 1..B
  int K;
  int N;
  int waves;       // W
  int bpw_log2;    // blocks per wave and phase = 1 << bpw_log2 (1, 2 or 4)
  int phases;      // ceil(K/256 / (W*bpw))
  int base_rows;   // N / gridDim.x; the first N % gridDim.x workgroups own one row more
  uint32_t w_bytes;   // N * row bytes, rounded up to a multiple of 4
  int32_t* dots_out;  // verification kernels only: int32 [rows, N, K/32] (Q6_K: K/16, signed dots), as block_dots writes them
};

constexpr int PSLAB_GROUP_ROWS = 96;

template <int QT>
struct PslabTraits;
template <>
struct PslabTraits<GGML_Q6_K> {
  static constexpr int BLK = Q6_K_BYTES;        // bytes per 256 values
  static constexpr int CPR = 14;                // 16-byte chunks loaded per row and block (224 bytes)
  static constexpr int PITCH = 240;             // LDS row pitch: 4 x 15 dwords
  static constexpr int REC_SLOT = 256 + 512;    // xd[8][8] floats, -32*qsum16[16][8] ints
};
template <>
struct PslabTraits<GGML_Q4_K> {
  static constexpr int BLK = Q4_K_BYTES;        // 144: 16-byte aligned rows, 9 chunks
  static constexpr int CPR = 9;
  static constexpr int PITCH = 144;             // 4 x 9 dwords
  static constexpr int REC_SLOT = 256 + 256;    // xd[8][8] floats, xd*qsum32[8][8] floats
};
template <>
struct PslabTraits<GGML_Q5_K> {
  static constexpr int BLK = Q5_K_BYTES;        // 176: 16-byte aligned rows, 11 chunks
  static constexpr int CPR = 11;
  static constexpr int PITCH = 176;             // 4 x 11 dwords
  static constexpr int REC_SLOT = 256 + 256;    // as Q4_K
};
template <>
struct PslabTraits<GGML_Q8_0> {
  static constexpr int BLK = 8 * Q8_0_BYTES;    // 272
  static constexpr int CPR = 17;
  static constexpr int PITCH = 272;             // 4 x 17 dwords
  static constexpr int REC_SLOT = 256;          // xd[8][8] floats
};

// LDS of one wave: the weight image of a unit (reused for the partial sums of a row group), a
// 16-byte dump slot, the per-block scale records and the int8 activations [B][bpw*256 + 16].
template <int QT>
constexpr int pslab_wave_bytes(int B, int bpw) {
  return 32 * PslabTraits<QT>::PITCH + 16 + bpw * PslabTraits<QT>::REC_SLOT + B * (bpw * 256 + 16);
}

// XK fixes the activation kind at compile time: the staging code of the other kinds is then not
// generated (it is most of the kernel's code, and cold instruction fetch is launch latency).
// DUMP: the verification instantiation, which also writes every int32 sub-block dot to a.dots_out.
template <int QT, int B, bool PHASED, int XK, bool DUMP = false>
__device__ __forceinline__ void gemv_pslab_workgroup(const GemvPslabArgs& a, uint8_t* smem) {
  using T = PslabTraits<QT>;
  constexpr int VB = B < 4 ? B : 4;
  constexpr int BLK = T::BLK, CPR = T::CPR, PITCH = T::PITCH;
  constexpr int RPI = 64 / CPR;                      // rows per wave-wide load: 4 (Q6_K), 3 (Q8_0)
  constexpr int NL = (32 + RPI - 1) / RPI;           // 16-byte loads per lane and unit
  constexpr int MAX_STEPS = PSLAB_GROUP_ROWS / 32;
  static_assert(B * PSLAB_GROUP_ROWS * 4 <= 32 * PITCH, "partial sums must fit the weight image");

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 31, g = lane >> 5;
  const int nb = a.K / QK_K;
  const int W = a.waves, bl2 = a.bpw_log2, bpw = 1 << bl2;
  const int row_bytes = nb * BLK;

  // rows of this workgroup
  const int wg = static_cast<int>(blockIdx.x), nwg = static_cast<int>(gridDim.x);
  const int extra = a.N - a.base_rows * nwg;
  const int r_begin = wg * a.base_rows + min(wg, extra);
  const int nrows = a.base_rows + (wg < extra ? 1 : 0);
  if (nrows <= 0) return;   // uniform over the workgroup

  // blocks of this wave: owned block j is block kb_of(j); nown of them are inside K
  // (slot s of phase p is block (p*bpw + s)*W + wave: the waves take the blocks of a phase round robin, so
  // 20 blocks over 12 waves x 2 slots give eight waves two blocks and four waves one - five per SIMD - and
  // the blocks a wave owns are a prefix of its slots)
  auto kb_of = [&](int j) { return j * W + wave; };
  int nown = 0;
  for (int j = 0; j < (a.phases << bl2); ++j) nown += kb_of(j) < nb ? 1 : 0;

  const int wave_bytes = pslab_wave_bytes<QT>(B, bpw);
  const int XQ_PITCH = bpw * 256 + 16;
  uint8_t* stage = smem + wave * wave_bytes;
  uint8_t* rec = stage + 32 * PITCH + 16;
  uint8_t* xq = rec + bpw * T::REC_SLOT;

  // ---- quantize the activations of owned blocks j0 .. j0+bpw-1 into xq / rec: 4 lanes per 32-value
  // group, 8 values per lane, 16 groups per pass; group id = (batch row, slot, sub-block)
  auto stage_x = [&](int j0) {
    constexpr int PCH = PHASED ? (QT == GGML_Q8_0 ? 2 : 4) : 8;                 // passes whose loads are in flight together
    // inside the main loop the lane's positions are recomputed on every call: hoisted out of the
    // loop they would stay in registers across the MFMA code, which has none to spare
    int lane_here = lane;
    if constexpr (PHASED) asm volatile("" : "+v"(lane_here));
    const int quad = lane_here >> 2, e = lane_here & 3;
    const int groups = B << (3 + bl2);
    for (int p0 = 0; p0 * 16 < groups; p0 += PCH) {
      uint32_t raw[PCH][8];
#pragma unroll
      for (int p = 0; p < PCH; ++p) {
        const int gid = (p0 + p) * 16 + quad;
        const int b = min(gid >> (3 + bl2), a.rows - 1);     // clamped: rows past the batch are zeroed below
        const int rem = gid & ((8 << bl2) - 1);
        const int jj = min(j0 + (rem >> 3), nown - 1);       // clamped: slots past the slice are not used
        const int col = kb_of(jj) * 8 + (rem & 7);           // 32-value group of the row
#pragma unroll
        for (int i = 0; i < 8; ++i) raw[p][i] = 0u;
        if ((p0 + p) * 16 >= groups) {
          // past the last pass
        } else if (XK == KIND_F32) {
          const uint4* src = reinterpret_cast<const uint4*>(static_cast<const float*>(a.x) + static_cast<int64_t>(b) * a.K + col * 32 + e * 8);
          const uint4 lo = src[0], hi = src[1];
          raw[p][0] = lo.x; raw[p][1] = lo.y; raw[p][2] = lo.z; raw[p][3] = lo.w;
          raw[p][4] = hi.x; raw[p][5] = hi.y; raw[p][6] = hi.z; raw[p][7] = hi.w;
        } else if (XK == KIND_Q8_1) {
          const uint8_t* blk = static_cast<const uint8_t*>(a.x) + (static_cast<int64_t>(b) * (a.K / 32) + col) * Q8_1_BYTES;
          raw[p][0] = *reinterpret_cast<const uint32_t*>(blk + 4 + 8 * e);
          raw[p][1] = *reinterpret_cast<const uint32_t*>(blk + 8 + 8 * e);
          raw[p][2] = *reinterpret_cast<const uint32_t*>(blk);
        } else {
          const uint4 h = *reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(a.x) + static_cast<int64_t>(b) * a.K + col * 32 + e * 8);
          raw[p][0] = h.x; raw[p][1] = h.y; raw[p][2] = h.z; raw[p][3] = h.w;
        }
      }
#pragma unroll
      for (int p = 0; p < PCH; ++p) {
        const int gid = (p0 + p) * 16 + quad;
        if ((p0 + p) * 16 >= groups) continue;
        const int b = gid >> (3 + bl2);                      // < B
        const int rem = gid & ((8 << bl2) - 1);
        const int slot = rem >> 3, sub = rem & 7;
        uint32_t packed[2];
        float xd;
        q8_quantize8(XK, raw[p], true, packed, xd);
        const bool used = b < a.rows && j0 + slot < nown;
        packed[0] = used ? packed[0] : 0u;
        packed[1] = used ? packed[1] : 0u;
        xd = used ? xd : 0.0f;
        *reinterpret_cast<uint2*>(xq + b * XQ_PITCH + slot * 256 + sub * 32 + e * 8) = make_uint2(packed[0], packed[1]);
        float* xdp = reinterpret_cast<float*>(rec + slot * T::REC_SLOT);
        if (e == 0) xdp[sub * 8 + b] = xd;
        if constexpr (QT == GGML_Q6_K) {
          int part = dot4(0x01010101u, packed[1], dot4(0x01010101u, packed[0], 0));
          part += dpp_i<DPP_QUAD_XOR1>(part);                // lanes 0,1: values 0..15; lanes 2,3: values 16..31
          int* s16 = reinterpret_cast<int*>(rec + slot * T::REC_SLOT + 256);
          if ((e & 1) == 0) s16[(2 * sub + (e >> 1)) * 8 + b] = -32 * part;
        } else if constexpr (QT == GGML_Q4_K || QT == GGML_Q5_K) {
          int total = dot4(0x01010101u, packed[1], dot4(0x01010101u, packed[0], 0));
          total += dpp_i<DPP_QUAD_XOR1>(total);
          total += dpp_i<DPP_QUAD_XOR2>(total);
          if (e == 0) xdp[64 + sub * 8 + b] = xd * static_cast<float>(total);
        }
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  };

  // ---- 16-byte chunks of a unit: lane l takes column l % CPR of rows i*RPI + l / CPR, i = 0..NL-1 (RPI rows per
  // wave-wide load; lanes past RPI*CPR idle).  A lane's load offsets then differ by a constant from load to
  // load and its LDS addresses by an immediate.
  const int r4 = lane / CPR, col16 = (lane - r4 * CPR) * 16;
  const bool loader = r4 < RPI;
  // Q6_K: a 210-byte block is 13 chunks and 2 bytes (the fp16 d).  The loads start at the block itself
  // (2-byte aligned buffer loads run at full rate; a 16-byte LDS read that is not 4-byte aligned takes a
  // cycle per lane), and the 14th chunk is the block's last 16 bytes, [194, 210), so that no load leaves
  // the row: its top half word, d, is stored as the first word of LDS chunk 13.
  const bool tail13 = QT == GGML_Q6_K && col16 == 13 * 16;
  const int goff = tail13 ? BLK - 16 : col16;
  const __amdgpu_buffer_rsrc_t wrsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(a.w), 0, a.w_bytes, 0x00020000);
  ps_u32x4 buf[NL];
  // unit (owned block j, step t) of the row group that starts at row g0 and has grows rows.  The whole
  // offset goes through the lane offset, which is the one the descriptor's range check sees.  Rows past
  // the group's last are clamped to it (their results are dropped), which keeps a ragged step from
  // reading rows of other workgroups.
  auto issue = [&](int j, int t, int g0, int grows) {
    const int last = min(grows - 32 * t - 1, 31);           // >= 0
    const uint32_t base = static_cast<uint32_t>(r_begin + g0 + 32 * t) * static_cast<uint32_t>(row_bytes) +
                          static_cast<uint32_t>(kb_of(j) * BLK) + static_cast<uint32_t>(goff);
    if (loader) {
      if (last == 31) {
        uint32_t off = base + static_cast<uint32_t>(__mul24(r4, row_bytes));
#pragma unroll
        for (int i = 0; i < NL; ++i) {
          const uint32_t o = (i + 1) * RPI <= 32 ? off : base + static_cast<uint32_t>(__mul24(min(i * RPI + r4, 31), row_bytes));
          buf[i] = __builtin_amdgcn_raw_buffer_load_b128(wrsrc, static_cast<int>(o), 0, 0);
          off += static_cast<uint32_t>(RPI * row_bytes);
        }
      } else {
#pragma unroll
        for (int i = 0; i < NL; ++i) {
          buf[i] = __builtin_amdgcn_raw_buffer_load_b128(
              wrsrc, static_cast<int>(base + static_cast<uint32_t>(__mul24(min(i * RPI + r4, last), row_bytes))), 0, 0);
        }
      }
    }
  };
  auto to_lds = [&]() {
    if (loader) {
      uint8_t* dst = stage + r4 * PITCH + col16;
#pragma unroll
      for (int i = 0; i < NL; ++i) {
        if constexpr (QT == GGML_Q6_K) buf[i].x = tail13 ? buf[i].w >> 16 : buf[i].x;
        if ((i + 1) * RPI <= 32 || i * RPI + r4 < 32) *reinterpret_cast<ps_u32x4*>(dst + i * RPI * PITCH) = buf[i];
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  };

  // to the wave's next unit (o, i) of the row group at g0u; g0u >= nrows afterwards: there is none
  auto advance = [&](int& o, int& i, int& g0u) {
    const int st = (min(PSLAB_GROUP_ROWS, nrows - g0u) + 31) >> 5;
    const int no = PHASED ? nown : st, ni = PHASED ? st : nown;
    if (i + 1 < ni) { ++i; }
    else if (o + 1 < no) { ++o; i = 0; }
    else { o = 0; i = 0; g0u += PSLAB_GROUP_ROWS; }
  };

  // ---- one unit: weights of block kb (image in `stage`) x activations of slot -> acc[v] for batch rows 4g+v
  // (row0, rows_here: first output row of the unit's step and how many of its 32 rows exist; DUMP only)
  auto compute = [&](int slot, int kb, float (&acc)[VB], int row0, int rows_here) {
    auto dump = [&](int index, int per_row, int v, int value) {
      const int m = 4 * g + v;
      if (m < a.rows && n < rows_here)
        a.dots_out[(static_cast<int64_t>(m) * a.N + row0 + n) * per_row + index] = value;
    };
    (void)dump;
    const uint8_t* xl = xq + min(n, B - 1) * XQ_PITCH + slot * 256;     // A operand row (rows >= B: results dropped)
    const float* xdp = reinterpret_cast<const float*>(rec + slot * T::REC_SLOT);
#pragma unroll
    for (int v = 0; v < VB; ++v) acc[v] = 0.0f;
    if constexpr (QT == GGML_Q6_K) {
      const uint8_t* wl = stage + n * PITCH;
      const int* s16 = reinterpret_cast<const int*>(rec + slot * T::REC_SLOT + 256);
      const uint4 scw = load16(wl + 192);
      ps_v16i zero16;
#pragma unroll
      for (int v = 0; v < 16; ++v) zero16[v] = 0;
      const float d = f16_bits_to_float(load2(wl + 208));
      // Software pipeline over the eight 32-value groups: the LDS reads of group k+1 (and of the second
      // half's weights) are in flight while the MFMAs and the scale arithmetic of group k run.
      // (The phased kernels hold the staging registers as well and read each group's operands when it is due.)
      constexpr bool PIPE = !PHASED;
      struct Wq { uint2 qa[2], qb[2], qh[2]; };
      struct Act { uint2 xv[2]; ps_v4i cs[2]; ps_f4 xd; };
      auto load_w = [&](int h) {
        Wq w;
#pragma unroll
        for (int l = 0; l < 2; ++l) {
          w.qa[l] = load8(wl + 64 * h + 16 * l + 8 * g);
          w.qb[l] = load8(wl + 64 * h + 32 + 16 * l + 8 * g);
          w.qh[l] = load8(wl + 128 + 32 * h + 16 * l + 8 * g);
        }
        return w;
      };
      auto load_act = [&](int j32) {
        Act t;
#pragma unroll
        for (int l = 0; l < 2; ++l) {
          t.xv[l] = *reinterpret_cast<const uint2*>(xl + 16 * (2 * j32 + l) + 8 * g);
          t.cs[l] = *reinterpret_cast<const ps_v4i*>(s16 + (2 * j32 + l) * 8 + 4 * g);   // -32 * qsum16 of rows 4g..4g+3
        }
        t.xd = *reinterpret_cast<const ps_f4*>(xdp + j32 * 8 + 4 * g);                   // xd of rows 4g..4g+3
        return t;
      };
      Wq wq[2];
      wq[0] = load_w(0);
      Act act = load_act(0);
#pragma unroll
      for (int j32 = 0; j32 < 8; ++j32) {                   // 32-value group of the block
        const int h = j32 >> 2, q = j32 & 3;
        Act act_next = act;
        if constexpr (PIPE) {
          if (j32 + 1 < 8) act_next = load_act(j32 + 1);
          if (j32 == 1) wq[1] = load_w(1);
        }
        int dots[2][VB];
#pragma unroll
        for (int l = 0; l < 2; ++l) {                       // 16-value group 2*j32 + l: scale index
          const Q6KQuad ux = q6k_unpack(wq[h].qa[l].x, wq[h].qb[l].x, wq[h].qh[l].x);
          const Q6KQuad uy = q6k_unpack(wq[h].qa[l].y, wq[h].qb[l].y, wq[h].qh[l].y);
          const uint32_t wx = q == 0 ? ux.g0 : q == 1 ? ux.g1 : q == 2 ? ux.g2 : ux.g3;
          const uint32_t wy = q == 0 ? uy.g0 : q == 1 ? uy.g1 : q == 2 ? uy.g2 : uy.g3;
          const long wop = static_cast<long>(static_cast<uint64_t>(wx) | (static_cast<uint64_t>(wy) << 32));
          const long xop = static_cast<long>(static_cast<uint64_t>(act.xv[l].x) | (static_cast<uint64_t>(act.xv[l].y) << 32));
          const ps_v16i r = __builtin_amdgcn_mfma_i32_32x32x16_i8(xop, wop, zero16, 0, 0, 0);
#pragma unroll
          for (int v = 0; v < VB; ++v) dots[l][v] = r[v] + act.cs[l][v];   // signed dot: sum x*(u - 32)
          if constexpr (DUMP) {
#pragma unroll
            for (int v = 0; v < VB; ++v) dump(kb * 16 + 2 * j32 + l, a.K / 16, v, dots[l][v]);
          }
        }
        const uint32_t sw = j32 < 2 ? scw.x : j32 < 4 ? scw.y : j32 < 6 ? scw.z : scw.w;
        const int sc0 = static_cast<int>(sw << (16 - 16 * (j32 & 1) + 8)) >> 24;   // int8 scale of group 2*j32
        const int sc1 = static_cast<int>(sw << (16 - 16 * (j32 & 1))) >> 24;       // int8 scale of group 2*j32+1
#pragma unroll
        for (int v = 0; v < VB; ++v) {
          // |dot| <= 16*127*32 < 2^23 and |sc| <= 128: 24-bit multiplies, exact sum
          const int iv = __mul24(dots[0][v], sc0) + __mul24(dots[1][v], sc1);
          acc[v] = __builtin_fmaf(act.xd[v], static_cast<float>(iv), acc[v]);
        }
        if constexpr (!PIPE) {
          if (j32 + 1 < 8) act_next = load_act(j32 + 1);
          if (j32 == 3) wq[1] = load_w(1);
        }
        act = act_next;
      }
#pragma unroll
      for (int v = 0; v < VB; ++v) acc[v] *= d;
    } else if constexpr (QT == GGML_Q4_K || QT == GGML_Q5_K) {
      // v_mfma_i32_32x32x32_i8 per 32-value sub-block; t = (d*sc) * float(dot), acc = fma(xd, t, acc),
      // acc = fma(-dmin*mn, xd*qsum, acc) (the arithmetic of gguf_q4_k_gemv.hip:893-904).  Q5_K: the same
      // with bit 4 of sub-block s, value l taken from bit s of qh[l] (gguf_k_gemv.hip:115-137).
      constexpr int QS = QT == GGML_Q5_K ? 48 : 16;      // offset of the nibbles
      const uint8_t* wl = stage + n * PITCH;
      ps_u32x4 qh = ps_u32x4{0u, 0u, 0u, 0u};
      if constexpr (QT == GGML_Q5_K) qh = *reinterpret_cast<const ps_u32x4*>(wl + 16 + 16 * g);   // qh[16g .. 16g+15]
      const ps_u32x4 hd = *reinterpret_cast<const ps_u32x4*>(wl);
      const Q4KScales u = q4k_unpack_scales(hd.y, hd.z, hd.w);
      const float d = f16_bits_to_float(hd.x & 0xFFFFu);
      const float dmin = f16_bits_to_float(hd.x >> 16);
      ps_v16i zero16;
#pragma unroll
      for (int v = 0; v < 16; ++v) zero16[v] = 0;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const ps_u32x4 qs = *reinterpret_cast<const ps_u32x4*>(wl + QS + 32 * j + 16 * g);
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          const int sb = 2 * j + half;
          ps_v4i wop;
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            uint32_t wv = half == 0 ? q4k_low(qs[c]) : q4k_high(qs[c]);
            if constexpr (QT == GGML_Q5_K) wv |= ((qh[c] >> sb) & 0x01010101u) << 4;
            wop[c] = static_cast<int>(wv);
          }
          const ps_v4i xop = *reinterpret_cast<const ps_v4i*>(xl + sb * 32 + 16 * g);
          const ps_v16i r = __builtin_amdgcn_mfma_i32_32x32x32_i8(xop, wop, zero16, 0, 0, 0);
          if constexpr (DUMP) {
#pragma unroll
            for (int v = 0; v < VB; ++v) dump(kb * 8 + sb, a.K / 32, v, r[v]);
          }
          const ps_f4 xd4 = *reinterpret_cast<const ps_f4*>(xdp + sb * 8 + 4 * g);
          const ps_f4 xs4 = *reinterpret_cast<const ps_f4*>(xdp + 64 + sb * 8 + 4 * g);
          const uint32_t sc = ((sb < 4 ? u.sc_lo : u.sc_hi) >> (8 * (sb & 3))) & 0xFFu;
          const uint32_t mn = ((sb < 4 ? u.mn_lo : u.mn_hi) >> (8 * (sb & 3))) & 0xFFu;
          const float sw = d * static_cast<float>(sc);
          const float mw = -(dmin * static_cast<float>(mn));
#pragma unroll
          for (int v = 0; v < VB; ++v) {
            const float tv = sw * static_cast<float>(r[v]);   // |dot| < 2^24: one rounding
            acc[v] = __builtin_fmaf(xd4[v], tv, acc[v]);
            acc[v] = __builtin_fmaf(mw, xs4[v], acc[v]);
          }
        }
      }
    } else {
      const uint8_t* wl = stage + n * PITCH;
      constexpr bool PIPE = !PHASED;   // as above: operands of block i+1 in flight during block i
      struct Ops { uint4 wv; uint32_t dw; ps_v4i xop; ps_f4 xd; };
      auto load_ops = [&](int i) {
        Ops t;
        t.wv = load16(wl + Q8_0_BYTES * i + 2 + 16 * g);
        t.dw = load2(wl + Q8_0_BYTES * i);
        t.xop = *reinterpret_cast<const ps_v4i*>(xl + 32 * i + 16 * g);
        t.xd = *reinterpret_cast<const ps_f4*>(xdp + i * 8 + 4 * g);
        return t;
      };
      ps_v16i zero16;
#pragma unroll
      for (int v = 0; v < 16; ++v) zero16[v] = 0;
      Ops ops = load_ops(0);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        Ops ops_next = ops;
        if constexpr (PIPE) {
          if (i + 1 < 8) ops_next = load_ops(i + 1);
        }
        const float dw = f16_bits_to_float(ops.dw);
        const ps_v4i wop = ps_v4i{static_cast<int>(ops.wv.x), static_cast<int>(ops.wv.y), static_cast<int>(ops.wv.z),
                                  static_cast<int>(ops.wv.w)};
        const ps_v16i r = __builtin_amdgcn_mfma_i32_32x32x32_i8(ops.xop, wop, zero16, 0, 0, 0);
        if constexpr (DUMP) {
#pragma unroll
          for (int v = 0; v < VB; ++v) dump(kb * 8 + i, a.K / 32, v, r[v]);
        }
#pragma unroll
        for (int v = 0; v < VB; ++v) {
          const float tv = dw * static_cast<float>(r[v]);    // |dot| < 2^24: one rounding
          acc[v] = __builtin_fmaf(ops.xd[v], tv, acc[v]);
        }
        if constexpr (!PIPE) {
          if (i + 1 < 8) ops_next = load_ops(i + 1);
        }
        ops = ops_next;
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
  };

  // ---- main loop
  constexpr bool one_phase = !PHASED;
  {
    issue(0, 0, 0, min(PSLAB_GROUP_ROWS, nrows));
  }
  if (one_phase) stage_x(0);

  for (int g0 = 0; g0 < nrows; g0 += PSLAB_GROUP_ROWS) {
    const int grows = min(PSLAB_GROUP_ROWS, nrows - g0);
    const int steps = (grows + 31) >> 5;
    float done[MAX_STEPS][VB];
#pragma unroll
    for (int t = 0; t < MAX_STEPS; ++t)
#pragma unroll
      for (int v = 0; v < VB; ++v) done[t][v] = 0.0f;

    // Unit order: with one phase, step by step and block by block inside a step (the step's sum stays in
    // four registers); with several, block by block and step by step inside a block (a block's
    // activations are quantized once).
    const int n_out = PHASED ? nown : steps, n_in = PHASED ? steps : nown;
#pragma unroll 1
    for (int o = 0; o < n_out; ++o) {
      float part[VB];
#pragma unroll
      for (int v = 0; v < VB; ++v) part[v] = 0.0f;
#pragma unroll 1
      for (int i = 0; i < n_in; ++i) {
        const int j = PHASED ? o : i, t = PHASED ? i : o;
        if (PHASED && t == 0 && (j & (bpw - 1)) == 0) stage_x(j);
        to_lds();
        // the loads of the next unit: of this group, or the first of the next
        int o1 = o, i1 = i, g1 = g0;
        advance(o1, i1, g1);
        if (g1 < nrows) {
          issue(PHASED ? o1 : i1, PHASED ? i1 : o1, g1, min(PSLAB_GROUP_ROWS, nrows - g1));
        }
        float acc[VB];
        compute(j & (bpw - 1), kb_of(j), acc, r_begin + g0 + 32 * t, min(grows - 32 * t, 32));
        if constexpr (PHASED) {
#pragma unroll
          for (int u = 0; u < MAX_STEPS; ++u)
#pragma unroll
            for (int v = 0; v < VB; ++v) done[u][v] = (u == t) ? done[u][v] + acc[v] : done[u][v];
        } else {
#pragma unroll
          for (int v = 0; v < VB; ++v) part[v] += acc[v];
        }
      }
      if constexpr (!PHASED) {
#pragma unroll
        for (int u = 0; u < MAX_STEPS; ++u)
#pragma unroll
          for (int v = 0; v < VB; ++v) done[u][v] = (u == o) ? part[v] : done[u][v];
      }
    }

    // ---- K-slice reduction of the group: the wave's partial sums [batch row][96] replace its weight image
    float* red = reinterpret_cast<float*>(stage);
#pragma unroll
    for (int t = 0; t < MAX_STEPS; ++t) {
#pragma unroll
      for (int v = 0; v < VB; ++v) {
        const int m = 4 * g + v, rl = 32 * t + n;
        if (m < B && rl < grows) red[m * PSLAB_GROUP_ROWS + rl] = done[t][v];
      }
    }
    __syncthreads();
    for (int idx = tid; idx < a.rows * grows; idx += blockDim.x) {
      const int m = idx / grows, rl = idx - m * grows;
      float v = 0.0f;
      for (int s = 0; s < W; ++s) v += reinterpret_cast<const float*>(smem + s * wave_bytes)[m * PSLAB_GROUP_ROWS + rl];
      const int64_t oi = static_cast<int64_t>(m) * a.N + r_begin + g0 + rl;
      if (a.residual) v = round_to_kind(v, a.out_kind) + load_scalar(a.residual, oi, a.out_kind);
      if (a.gate) {   // the up half of a gate/up pair: the gate projection is already stored, rounded
        const float gt = load_scalar(a.gate, oi, a.out_kind);
        const float sig = 1.0f / (1.0f + expf(-gt));
        v = gt * sig * round_to_kind(v, a.out_kind);
      }
      store_scalar(a.out, oi, v, a.out_kind);
    }
    __syncthreads();
  }
}

}  // namespace hipengine_gfx950
