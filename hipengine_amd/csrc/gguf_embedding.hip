// Token embedding lookup over raw GGUF rows: out[r, :] = bf16(dequantize(qweight[token_ids[r], :])).
// Rows whose token id is outside [0, vocab_size) are left untouched, as in
// kernels/hip_gfx1100/quant/gguf_q6_k_embedding.hip:140-235.

#include "gguf_dequant.hpp"

#include "gguf_init.hpp"

#include "../../include/hipengine_gfx950.h"

namespace {

using namespace hipengine_gfx950;

// grid (ceil(units per row / 256), rows); one dequantization unit per thread.
template <int QT>
__global__ void __launch_bounds__(256) embedding_kernel(const int64_t* __restrict__ token_ids,
                                                        const uint8_t* __restrict__ qweight,
                                                        uint16_t* __restrict__ out, int hidden_size,
                                                        int64_t vocab_size) {
  using T = DequantTraits<QT>;
  const int row = blockIdx.y;
  const int64_t token = token_ids[row];
  if (token < 0 || token >= vocab_size) return;
  const int blocks_per_row = hidden_size / T::VALUES;
  const int unit = blockIdx.x * 256 + threadIdx.x;
  const int b = unit / T::UNITS;
  if (b >= blocks_per_row) return;
  const uint8_t* blk = qweight + (token * blocks_per_row + b) * T::BYTES;
  uint16_t* o = out + static_cast<int64_t>(row) * hidden_size + b * T::VALUES;
  dequant_unit<QT>(blk, unit - b * T::UNITS, [=](int k, float v) { o[k] = float_to_bf16_bits(v); });
}

template <int QT>
int launch_embedding(const int64_t* token_ids, const uint8_t* qweight, uint16_t* out, int64_t rows,
                     int64_t hidden_size, int64_t vocab_size, hipStream_t stream) {
  using T = DequantTraits<QT>;
  if (!token_ids || !qweight || !out || rows <= 0 || rows > 65535 || hidden_size <= 0 || vocab_size <= 0 ||
      (hidden_size % T::VALUES) != 0 || hidden_size > (1 << 24)) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  const int units = static_cast<int>(hidden_size / T::VALUES) * T::UNITS;
  const dim3 grid(static_cast<unsigned>((units + 255) / 256), static_cast<unsigned>(rows));
  hipLaunchKernelGGL(embedding_kernel<QT>, grid, dim3(256), 0, stream, token_ids, qweight, out,
                     static_cast<int>(hidden_size), vocab_size);
  return static_cast<int>(hipGetLastError());
}

}  // namespace

#define DEFINE_EMBEDDING(NAME, QT)                                                                          \
  extern "C" int hipengine_gguf_##NAME##_embedding_bf16_out(const int64_t* token_ids, const uint8_t* qweight, \
                                                            uint16_t* out, int64_t rows, int64_t hidden_size, \
                                                            int64_t vocab_size, int64_t threads,              \
                                                            hipStream_t stream) {                             \
    (void)threads;                                                                                            \
    return launch_embedding<QT>(token_ids, qweight, out, rows, hidden_size, vocab_size, stream);              \
  }

DEFINE_EMBEDDING(q4_k, GGML_Q4_K)
DEFINE_EMBEDDING(q5_k, GGML_Q5_K)
DEFINE_EMBEDDING(q6_k, GGML_Q6_K)
DEFINE_EMBEDDING(q8_0, GGML_Q8_0)

int hipengine_gfx950::embedding_load() {
  hipFuncAttributes attr;
  return static_cast<int>(hipFuncGetAttributes(&attr, reinterpret_cast<const void*>(embedding_kernel<GGML_Q4_K>)));
}
