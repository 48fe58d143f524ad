// Launch interface between the translation units of the decode GEMV: the dispatcher and C entry points
// (gguf_gemv.hip) and the kernel families, each compiled on its own (gguf_gemv_stream.hip,
// gguf_gemv_slab.hip, gguf_gemv_pslab.hip).  A plan says how a family would run a shape (`ok` false: it
// does not take it); launch_* validates the plan again and launches.  All return a hipError_t as int.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace hipengine_gfx950 {

constexpr size_t kMaxLds = 160 * 1024;   // LDS of one CU
constexpr int kComputeUnits = 256;       // MI355X

inline int batch_bucket(int rows) { return rows <= 1 ? 1 : rows <= 2 ? 2 : rows <= 4 ? 4 : 8; }

// ---- slab form (Q4_K on the int8 MFMA, one workgroup per CU, waves split K) ----
struct SlabPlan {
  int b, bpw, waves, two_block_waves, rows_wg;
  bool ok;
};
constexpr int SLAB_PAIR_ROWS = 72;   // rows per workgroup up to which the gate/up pair runs as one slab launch
SlabPlan default_slab_plan(int qt, int rows, int64_t K, int64_t N);
int launch_gemv_slab(const void* x, int x_kind, const uint8_t* w, void* out, int out_kind, int rows, int64_t K,
                     int64_t N, const SlabPlan& p, hipStream_t stream, const void* residual = nullptr,
                     const void* gate = nullptr, int32_t* dots_out = nullptr, const uint8_t* w_up = nullptr);
bool slab_multi_ok(int count, const int* qt, int rows, int64_t K, const int64_t* N);
int launch_gemv_slab_multi(int count, const void* x, int x_kind, const uint8_t* const* w, void* const* out, int out_kind,
                           int rows, int64_t K, const int64_t* N, hipStream_t stream);
int slab_raise_lds_limits();

// ---- phased slab form (int8 MFMA; batch 3..8) ----
struct PslabPlan {
  int b, waves, bpw_log2, phases, grid;
  bool ok;
};
PslabPlan default_pslab_plan(int qt, int rows, int64_t K, int64_t N, const void* w);
int pslab_grid(int64_t N, int phases);
int launch_gemv_pslab(int qt, const void* x, int x_kind, const uint8_t* w, void* out, int out_kind, int rows,
                      int64_t K, int64_t N, const PslabPlan& p, hipStream_t stream, const void* residual = nullptr,
                      const void* gate = nullptr, int32_t* dots_out = nullptr);
int pslab_raise_lds_limits();

// ---- direct slab form (weights streamed straight into LDS, int8 MFMA; batch 2..8) ----
struct DslabPlan {
  int waves, ring, row_groups, ksplit, blocks_part;
  bool ok;
};
DslabPlan default_dslab_plan(int qt, int rows, int64_t K, int64_t N, const void* w);
DslabPlan dslab_plan_for(int qt, int rows, int64_t K, int64_t N, const void* w, int parts);
int launch_gemv_dslab(int qt, const void* x, int x_kind, const uint8_t* w, void* out, int out_kind, int rows,
                      int64_t K, int64_t N, const DslabPlan& p, hipStream_t stream, const void* residual = nullptr,
                      const void* gate = nullptr, int32_t* dots_out = nullptr);
int dslab_setup(int device);   // per device: dynamic-LDS limits, addresses of the split-K scratch

// ---- stream form (resident waves, ring of loads in flight) ----
enum StreamFuse { FUSE_NONE = 0, FUSE_PAIR = 1, FUSE_RESIDUAL = 2, FUSE_DUAL = 3 };   // epilogue of the stream kernels
struct StreamPlan {
  int b, d, waves, waves_total;
  bool ok;
};
struct StreamFusion {
  int fuse = FUSE_NONE;
  const uint8_t* w_up = nullptr;
  const void* residual = nullptr;
  int round_mid = 0;
  void* out_b = nullptr;      // FUSE_DUAL
};
StreamPlan default_stream_plan(int qt, int rows, int64_t K, int64_t N, int fuse = FUSE_NONE);
int launch_gemv_stream(int qt, const void* x, int x_kind, const uint8_t* w, void* out, int out_kind, int rows,
                       int64_t K, int64_t N, const StreamPlan& p, hipStream_t stream,
                       const StreamFusion& fusion = StreamFusion());
// Up to four matrices of any supported types over one activation (rows <= 2), one launch.
bool stream_multi_ok(int count, const int* qt, int rows, int64_t K, const int64_t* N);
int launch_gemv_stream_multi(int count, const int* qt, const void* x, int x_kind, const uint8_t* const* w,
                             void* const* out, int out_kind, int rows, int64_t K, const int64_t* N,
                             hipStream_t stream);
int stream_raise_lds_limits();

}  // namespace hipengine_gfx950
