/*
 * CPU oracle for the GGUF k-quant matmul path, plain C.  TEST INFRASTRUCTURE ONLY.
 *
 * A scalar, loop-per-element restatement of (a) hipEngine's CPU reference
 * backend (dequantize the whole weight to float32, then a float32 matmul) and
 * (b) the device-side arithmetic specifications the gfx950 kernels are held
 * to: q8_1 activation quantizers, int32 sub-block dots and their float32
 * combination.  It exists so that the test-suite can check the HIP kernels and
 * so that the benchmark can time a CPU baseline; the shipped library never
 * links, loads or calls it.
 *
 * It is written independently of oracle/gguf_oracle.py (per-element index
 * maps here, vectorized reshapes there) and the tests pin the two against
 * each other and against the reference's own known answers.  The pinning
 * status of every function is listed in the header of gguf_oracle.py.
 *
 * Reference sources followed (paths relative to the hipEngine tree):
 *   hipengine/quant/gguf.py:604-681                      block dequantizers
 *   hipengine/kernels/cpu_reference/ops.py:466-484       dequant -> matmul GEMV
 *   hipengine/kernels/cpu_reference/ops.py:624-678       selected-expert MoE FFN
 *   kernels/hip_gfx1100/quant/gguf_q4_k_gemv.hip:74-106  Q4_K scale/min + element map
 *   kernels/hip_gfx1100/quant/gguf_q4_k_gemv.hip:740-772 q8_1 quantizer (GEMV convention)
 *   kernels/hip_gfx1100/quant/gguf_q4_k_gemv.hip:893-904 Q4_K x q8_1 combine
 *   kernels/hip_gfx1100/quant/gguf_k_gemv.hip:139-160,233-246   Q6_K element map, combine
 *   kernels/hip_gfx1100/quant/gguf_q8_0_dp4a_gemv.hip:100-137   Q8_0 x q8_1
 *   kernels/hip_gfx1100/quant/gguf_q4_k_q8_1_selected_prefill.hip:627-690  DS4 pack
 *   kernels/hip_gfx1100/quant/gguf_q4_k_q8_1_mmq_prefill.hip:158-289       Q4_K MMQ
 *   kernels/hip_gfx1100/quant/gguf_k_mmq_prefill.hip:264-307,519-685       D4S4, Q6_K MMQ
 */
#include <math.h>
#ifdef _OPENMP
#include <omp.h>
#endif
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define QK_K 256
#define Q4_K_BYTES 144
#define Q6_K_BYTES 210
#define Q8_0_BYTES 34
#define Q8_1_BYTES 36
#define DS4_BYTES 144
#define D4S4_BYTES 160

/* ---- fp16 / bf16 ------------------------------------------------------- */

float oracle_f16_to_f32(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  const uint32_t exp = (h >> 10) & 0x1Fu;
  uint32_t man = h & 0x3FFu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else { /* subnormal: normalize */
      int e = -1;
      do { man <<= 1; ++e; } while ((man & 0x400u) == 0);
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3FFu) << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7F800000u | (man << 13);
  } else {
    bits = sign | ((exp + 112u) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

/* round-to-nearest-even float32 -> fp16, subnormals and overflow to inf included */
uint16_t oracle_f32_to_f16(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  const uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
  const uint32_t absx = x & 0x7FFFFFFFu;
  if (absx >= 0x7F800000u) { /* inf / nan */
    return (uint16_t)(sign | 0x7C00u | ((absx > 0x7F800000u) ? 0x200u : 0u));
  }
  if (absx >= 0x477FF000u) { /* >= 65520 rounds to inf */
    return (uint16_t)(sign | 0x7C00u);
  }
  if (absx < 0x38800000u) { /* below smallest normal half (2^-14) */
    if (absx < 0x33000000u) return sign; /* < 2^-25 rounds to zero */
    const int e = (int)(absx >> 23);
    const uint32_t man = (absx & 0x7FFFFFu) | 0x800000u;
    const int shift = 126 - e; /* bits to drop so that unit = 2^-24 */
    const uint32_t q = man >> shift;
    const uint32_t rem = man & ((1u << shift) - 1u);
    const uint32_t half = 1u << (shift - 1);
    uint32_t r = q;
    if (rem > half || (rem == half && (q & 1u))) ++r;
    return (uint16_t)(sign | r);
  }
  const uint32_t e = (absx >> 23) - 112u;
  const uint32_t man = absx & 0x7FFFFFu;
  uint32_t r = (e << 10) | (man >> 13);
  const uint32_t rem = man & 0x1FFFu;
  if (rem > 0x1000u || (rem == 0x1000u && (r & 1u))) ++r;
  return (uint16_t)(sign | r);
}

static inline float bf16_to_f32(uint16_t b) {
  const uint32_t bits = (uint32_t)b << 16;
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

uint16_t oracle_f32_to_bf16(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  x += 0x7FFFu + ((x >> 16) & 1u);
  return (uint16_t)(x >> 16);
}

static inline float rd_f16(const uint8_t* p) {
  return oracle_f16_to_f32((uint16_t)(p[0] | (p[1] << 8)));
}

static inline void wr_f16(uint8_t* p, float v) {
  const uint16_t h = oracle_f32_to_f16(v);
  p[0] = (uint8_t)(h & 0xFF);
  p[1] = (uint8_t)(h >> 8);
}

/* ---- per-element integer unpack ---------------------------------------- */

static inline int q4k_scale(const uint8_t* s, int j) {
  return j < 4 ? (s[j] & 63) : ((s[j + 4] & 0x0F) | ((s[j - 4] >> 2) & 0x30));
}

static inline int q4k_min(const uint8_t* s, int j) {
  return j < 4 ? (s[j + 4] & 63) : ((s[j + 4] >> 4) | ((s[j] >> 2) & 0x30));
}

/* unsigned nibble of element k (0..255) of one 144-byte block */
static inline int q4k_quant(const uint8_t* blk, int k) {
  const int sb = k >> 5, lane = k & 31;
  const uint8_t byte = blk[16 + (sb >> 1) * 32 + lane];
  return (sb & 1) ? (byte >> 4) : (byte & 0x0F);
}

/* signed 6-bit value (already minus 32) of element k of one 210-byte block */
static inline int q6k_quant(const uint8_t* blk, int k) {
  const int g = k >> 5, lane = k & 31;
  const uint8_t lb = blk[(g >= 4 ? 64 : 0) + (g & 1) * 32 + lane];
  const int low = (g & 2) ? (lb >> 4) : (lb & 0x0F);
  const int high = (blk[128 + (g >= 4 ? 32 : 0) + lane] >> (2 * (g & 3))) & 3;
  return (low | (high << 4)) - 32;
}

void oracle_q4_k_scale_min(const uint8_t* scale_bytes, int64_t n_blocks, uint8_t* sc, uint8_t* mn) {
  for (int64_t b = 0; b < n_blocks; ++b)
    for (int j = 0; j < 8; ++j) {
      sc[b * 8 + j] = (uint8_t)q4k_scale(scale_bytes + b * 12, j);
      mn[b * 8 + j] = (uint8_t)q4k_min(scale_bytes + b * 12, j);
    }
}

void oracle_q4_k_unpack_int(const uint8_t* blocks, int64_t n_blocks, uint8_t* q) {
  for (int64_t b = 0; b < n_blocks; ++b)
    for (int k = 0; k < QK_K; ++k) q[b * QK_K + k] = (uint8_t)q4k_quant(blocks + b * Q4_K_BYTES, k);
}

void oracle_q6_k_unpack_int(const uint8_t* blocks, int64_t n_blocks, int8_t* q) {
  for (int64_t b = 0; b < n_blocks; ++b)
    for (int k = 0; k < QK_K; ++k) q[b * QK_K + k] = (int8_t)q6k_quant(blocks + b * Q6_K_BYTES, k);
}

/* ---- dequantizers (float32, one rounding at most) ----------------------- */

void oracle_dequant_q4_k(const uint8_t* blocks, int64_t n_blocks, float* out) {
#pragma omp parallel for schedule(static)
  for (int64_t b = 0; b < n_blocks; ++b) {
    const uint8_t* blk = blocks + b * Q4_K_BYTES;
    const float d = rd_f16(blk), dmin = rd_f16(blk + 2);
    for (int sb = 0; sb < 8; ++sb) {
      const float scale = d * (float)q4k_scale(blk + 4, sb);
      const float minv = dmin * (float)q4k_min(blk + 4, sb);
      for (int lane = 0; lane < 32; ++lane) {
        const int k = sb * 32 + lane;
        out[b * QK_K + k] = scale * (float)q4k_quant(blk, k) - minv; /* the product is exact: one rounding */
      }
    }
  }
}

void oracle_dequant_q6_k(const uint8_t* blocks, int64_t n_blocks, float* out) {
#pragma omp parallel for schedule(static)
  for (int64_t b = 0; b < n_blocks; ++b) {
    const uint8_t* blk = blocks + b * Q6_K_BYTES;
    const float d = rd_f16(blk + 208);
    const int8_t* sc = (const int8_t*)(blk + 192);
    for (int k = 0; k < QK_K; ++k) out[b * QK_K + k] = (d * (float)sc[k >> 4]) * (float)q6k_quant(blk, k);
  }
}

void oracle_dequant_q8_0(const uint8_t* blocks, int64_t n_blocks, float* out) {
#pragma omp parallel for schedule(static)
  for (int64_t b = 0; b < n_blocks; ++b) {
    const uint8_t* blk = blocks + b * Q8_0_BYTES;
    const float d = rd_f16(blk);
    for (int k = 0; k < 32; ++k) out[b * 32 + k] = (float)((const int8_t*)(blk + 2))[k] * d;
  }
}

static int64_t type_bytes(int qtype) { return qtype == 12 ? Q4_K_BYTES : qtype == 14 ? Q6_K_BYTES : Q8_0_BYTES; }
static int64_t type_block(int qtype) { return qtype == 8 ? 32 : QK_K; }

static void dequant_rows(const uint8_t* w, int qtype, int64_t n_blocks, float* out) {
  if (qtype == 12) oracle_dequant_q4_k(w, n_blocks, out);
  else if (qtype == 14) oracle_dequant_q6_k(w, n_blocks, out);
  else oracle_dequant_q8_0(w, n_blocks, out);
}

/*
 * CPU reference backend GEMV: out[r,n] = sum_k x[r,k] * dequant(W)[n,k], float32
 * inputs, accumulated here in double so the result is the correctly rounded
 * value any float32 summation order is compared against.  Weight rows are
 * dequantized `chunk` at a time.  Returns 0, or -1 on allocation failure.
 */
int oracle_gemv_dequant(const float* x, const uint8_t* w, int qtype, float* out,
                        int64_t rows, int64_t in_features, int64_t out_features) {
  const int64_t bpr = in_features / type_block(qtype);
  const int64_t row_bytes = bpr * type_bytes(qtype);
  const int64_t chunk = 1024;
  float* buf = (float*)malloc((size_t)chunk * (size_t)in_features * sizeof(float));
  if (!buf) return -1;
  for (int64_t n0 = 0; n0 < out_features; n0 += chunk) {
    const int64_t n1 = n0 + chunk < out_features ? n0 + chunk : out_features;
    dequant_rows(w + n0 * row_bytes, qtype, (n1 - n0) * bpr, buf);
#pragma omp parallel for schedule(static)
    for (int64_t n = n0; n < n1; ++n) {
      const float* wr = buf + (n - n0) * in_features;
      for (int64_t r = 0; r < rows; ++r) {
        double acc = 0.0;
        const float* xr = x + r * in_features;
        for (int64_t k = 0; k < in_features; ++k) acc += (double)xr[k] * (double)wr[k];
        out[r * out_features + n] = (float)acc;
      }
    }
  }
  free(buf);
  return 0;
}

/* ---- activation quantizers --------------------------------------------- */

static float tree_sum32(const float* v) { /* 32-lane shfl_down tree: +16,+8,+4,+2,+1 */
  float t[32];
  memcpy(t, v, sizeof t);
  for (int w = 16; w >= 1; w >>= 1)
    for (int i = 0; i < w; ++i) t[i] = t[i] + t[i + w];
  return t[0];
}

static void quantize_q8_1_block(const float* v, uint8_t* dst) {
  float amax = 0.0f;
  for (int i = 0; i < 32; ++i) amax = fmaxf(amax, fabsf(v[i]));
  const float d = amax / 127.0f;
  for (int i = 0; i < 32; ++i) {
    int q = (amax == 0.0f) ? 0 : (int)roundf(v[i] / d);
    q = q < -128 ? -128 : (q > 127 ? 127 : q);
    dst[4 + i] = (uint8_t)(int8_t)q;
  }
  wr_f16(dst, d);
  wr_f16(dst + 2, tree_sum32(v));
}

void oracle_quantize_q8_1_f32(const float* x, uint8_t* xq, int64_t rows, int64_t in_features) {
  const int64_t nb = in_features / 32;
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < rows * nb; ++i) quantize_q8_1_block(x + i * 32, xq + i * Q8_1_BYTES);
}

void oracle_quantize_q8_1_bf16(const uint16_t* x, uint8_t* xq, int64_t rows, int64_t in_features) {
  const int64_t nb = in_features / 32;
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < rows * nb; ++i) {
    float v[32];
    for (int j = 0; j < 32; ++j) v[j] = bf16_to_f32(x[i * 32 + j]);
    quantize_q8_1_block(v, xq + i * Q8_1_BYTES);
  }
}

void oracle_pack_ds4_bf16(const uint16_t* x, uint8_t* out, int64_t rows, int64_t hidden) {
  const int64_t nb = hidden / 128;
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < rows * nb; ++i) {
    uint8_t* dst = out + i * DS4_BYTES;
    for (int g = 0; g < 4; ++g) {
      float v[32];
      float amax = 0.0f;
      for (int j = 0; j < 32; ++j) {
        v[j] = bf16_to_f32(x[i * 128 + g * 32 + j]);
        amax = fmaxf(amax, fabsf(v[j]));
      }
      const float scale = fminf(65504.0f, amax / 127.0f);
      const float sum = fminf(65504.0f, fmaxf(-65504.0f, tree_sum32(v)));
      for (int j = 0; j < 32; ++j) {
        int q = 0;
        if (scale > 0.0f) q = (int)fminf(127.0f, fmaxf(-127.0f, rintf(v[j] / scale)));
        dst[16 + g * 32 + j] = (uint8_t)(int8_t)q;
      }
      wr_f16(dst + 4 * g, scale);
      wr_f16(dst + 4 * g + 2, sum);
    }
  }
}

void oracle_pack_d4s4_bf16(const uint16_t* x, uint8_t* out, int64_t rows, int64_t hidden) {
  const int64_t nb = hidden / 128;
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < rows * nb; ++i) {
    uint8_t* dst = out + i * D4S4_BYTES;
    for (int g = 0; g < 4; ++g) {
      float v[32], part[8];
      float amax = 0.0f;
      for (int j = 0; j < 32; ++j) {
        v[j] = bf16_to_f32(x[i * 128 + g * 32 + j]);
        amax = fmaxf(amax, fabsf(v[j]));
      }
      for (int t = 0; t < 8; ++t) {
        float s = 0.0f;
        for (int e = 0; e < 4; ++e) s += v[4 * t + e];
        part[t] = s;
      }
      for (int w = 4; w >= 1; w >>= 1)
        for (int t = 0; t < w; ++t) part[t] = part[t] + part[t + w];
      const float d = amax == 0.0f ? 0.0f : amax / 127.0f;
      for (int j = 0; j < 32; ++j) {
        int q = d == 0.0f ? 0 : (int)roundf(v[j] / d);
        q = q < -128 ? -128 : (q > 127 ? 127 : q);
        dst[32 + g * 32 + j] = (uint8_t)(int8_t)q;
      }
      memcpy(dst + 4 * g, &d, 4);
      memcpy(dst + 16 + 4 * g, &part[0], 4);
    }
  }
}

/* ---- int32 sub-block dots ---------------------------------------------- */

/* dots[r][n][j] = sum_{i<32} q4[n][32j+i] * q8[r][32j+i];  qsum[r][j] = sum q8.
 * xq: 36-byte q8_1 blocks [rows][K/32]. */
void oracle_q4_k_q8_1_block_dots(const uint8_t* xq, const uint8_t* w, int32_t* dots, int32_t* qsum,
                                 int64_t rows, int64_t in_features, int64_t out_features) {
  const int64_t nsb = in_features / 32, row_bytes = in_features / QK_K * Q4_K_BYTES;
  for (int64_t r = 0; r < rows; ++r)
    for (int64_t j = 0; j < nsb; ++j) {
      const int8_t* q8 = (const int8_t*)(xq + (r * nsb + j) * Q8_1_BYTES + 4);
      int32_t s = 0;
      for (int i = 0; i < 32; ++i) s += q8[i];
      qsum[r * nsb + j] = s;
    }
#pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < out_features; ++n)
    for (int64_t r = 0; r < rows; ++r)
      for (int64_t j = 0; j < nsb; ++j) {
        const uint8_t* blk = w + n * row_bytes + (j >> 3) * Q4_K_BYTES;
        const int8_t* q8 = (const int8_t*)(xq + (r * nsb + j) * Q8_1_BYTES + 4);
        int32_t acc = 0;
        for (int i = 0; i < 32; ++i) acc += q4k_quant(blk, (int)(j & 7) * 32 + i) * (int32_t)q8[i];
        dots[(r * out_features + n) * nsb + j] = acc;
      }
}

/* dots[r][n][j16] = sum_{i<16} (u6-32)[n][16j+i] * q8[r][16j+i] */
void oracle_q6_k_q8_1_block_dots(const uint8_t* xq, const uint8_t* w, int32_t* dots,
                                 int64_t rows, int64_t in_features, int64_t out_features) {
  const int64_t n16 = in_features / 16, nsb = in_features / 32, row_bytes = in_features / QK_K * Q6_K_BYTES;
#pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < out_features; ++n)
    for (int64_t r = 0; r < rows; ++r)
      for (int64_t j = 0; j < n16; ++j) {
        const uint8_t* blk = w + n * row_bytes + (j >> 4) * Q6_K_BYTES;
        const int8_t* q8 = (const int8_t*)(xq + (r * nsb + (j >> 1)) * Q8_1_BYTES + 4) + (j & 1) * 16;
        int32_t acc = 0;
        for (int i = 0; i < 16; ++i) acc += q6k_quant(blk, (int)(j & 15) * 16 + i) * (int32_t)q8[i];
        dots[(r * out_features + n) * n16 + j] = acc;
      }
}

void oracle_q8_0_q8_1_block_dots(const uint8_t* xq, const uint8_t* w, int32_t* dots,
                                 int64_t rows, int64_t in_features, int64_t out_features) {
  const int64_t nsb = in_features / 32, row_bytes = nsb * Q8_0_BYTES;
#pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < out_features; ++n)
    for (int64_t r = 0; r < rows; ++r)
      for (int64_t j = 0; j < nsb; ++j) {
        const int8_t* wq = (const int8_t*)(w + n * row_bytes + j * Q8_0_BYTES + 2);
        const int8_t* q8 = (const int8_t*)(xq + (r * nsb + j) * Q8_1_BYTES + 4);
        int32_t acc = 0;
        for (int i = 0; i < 32; ++i) acc += (int32_t)wq[i] * (int32_t)q8[i];
        dots[(r * out_features + n) * nsb + j] = acc;
      }
}

/* ---- q8_1 GEMV in the device formula, float32 in sub-block order --------- */

void oracle_q4_k_q8_1_gemv(const uint8_t* xq, const uint8_t* w, float* out,
                           int64_t rows, int64_t in_features, int64_t out_features) {
  const int64_t nsb = in_features / 32, row_bytes = in_features / QK_K * Q4_K_BYTES;
#pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < out_features; ++n)
    for (int64_t r = 0; r < rows; ++r) {
      float acc = 0.0f;
      for (int64_t j = 0; j < nsb; ++j) {
        const uint8_t* blk = w + n * row_bytes + (j >> 3) * Q4_K_BYTES;
        const uint8_t* xb = xq + (r * nsb + j) * Q8_1_BYTES;
        const int8_t* q8 = (const int8_t*)(xb + 4);
        int32_t dot = 0, qs = 0;
        for (int i = 0; i < 32; ++i) {
          dot += q4k_quant(blk, (int)(j & 7) * 32 + i) * (int32_t)q8[i];
          qs += q8[i];
        }
        const float xd = rd_f16(xb);
        const float dsc = rd_f16(blk) * (float)q4k_scale(blk + 4, (int)(j & 7));
        const float dmn = rd_f16(blk + 2) * (float)q4k_min(blk + 4, (int)(j & 7));
        acc += xd * (dsc * (float)dot - dmn * (float)qs);
      }
      out[r * out_features + n] = acc;
    }
}

void oracle_q6_k_q8_1_gemv(const uint8_t* xq, const uint8_t* w, float* out,
                           int64_t rows, int64_t in_features, int64_t out_features) {
  const int64_t n16 = in_features / 16, nsb = in_features / 32, row_bytes = in_features / QK_K * Q6_K_BYTES;
#pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < out_features; ++n)
    for (int64_t r = 0; r < rows; ++r) {
      float acc = 0.0f;
      for (int64_t j = 0; j < n16; ++j) {
        const uint8_t* blk = w + n * row_bytes + (j >> 4) * Q6_K_BYTES;
        const uint8_t* xb = xq + (r * nsb + (j >> 1)) * Q8_1_BYTES;
        const int8_t* q8 = (const int8_t*)(xb + 4) + (j & 1) * 16;
        int32_t dot = 0;
        for (int i = 0; i < 16; ++i) dot += q6k_quant(blk, (int)(j & 15) * 16 + i) * (int32_t)q8[i];
        acc += rd_f16(xb) * rd_f16(blk + 208) * (float)((const int8_t*)(blk + 192))[j & 15] * (float)dot;
      }
      out[r * out_features + n] = acc;
    }
}

void oracle_q8_0_q8_1_gemv(const uint8_t* xq, const uint8_t* w, float* out,
                           int64_t rows, int64_t in_features, int64_t out_features) {
  const int64_t nsb = in_features / 32, row_bytes = nsb * Q8_0_BYTES;
#pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < out_features; ++n)
    for (int64_t r = 0; r < rows; ++r) {
      float acc = 0.0f;
      for (int64_t j = 0; j < nsb; ++j) {
        const uint8_t* wb = w + n * row_bytes + j * Q8_0_BYTES;
        const uint8_t* xb = xq + (r * nsb + j) * Q8_1_BYTES;
        int32_t dot = 0;
        for (int i = 0; i < 32; ++i) dot += (int32_t)((const int8_t*)(wb + 2))[i] * (int32_t)((const int8_t*)(xb + 4))[i];
        acc += rd_f16(wb) * rd_f16(xb) * (float)dot;
      }
      out[r * out_features + n] = acc;
    }
}

/* ---- MMQ in the device formula ------------------------------------------ */

/* acc += (d*sc)*xd*dot - (dmin*mn)*xsum per sub-block, float32, sub-block order.
 * xds4: 144-byte DS4 blocks [rows][K/128]. */
void oracle_q4_k_ds4_mmq(const uint8_t* xds4, const uint8_t* w, float* out,
                         int64_t rows, int64_t in_features, int64_t out_features) {
  const int64_t nsb = in_features / 32, row_bytes = in_features / QK_K * Q4_K_BYTES;
  const int64_t x_row_bytes = in_features / 128 * DS4_BYTES;
#pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < out_features; ++n)
    for (int64_t r = 0; r < rows; ++r) {
      float acc = 0.0f;
      for (int64_t j = 0; j < nsb; ++j) {
        const uint8_t* blk = w + n * row_bytes + (j >> 3) * Q4_K_BYTES;
        const uint8_t* xb = xds4 + r * x_row_bytes + (j >> 2) * DS4_BYTES;
        const int8_t* q8 = (const int8_t*)(xb + 16) + (j & 3) * 32;
        int32_t dot = 0;
        for (int i = 0; i < 32; ++i) dot += q4k_quant(blk, (int)(j & 7) * 32 + i) * (int32_t)q8[i];
        const float xd = rd_f16(xb + 4 * (j & 3)), xsum = rd_f16(xb + 4 * (j & 3) + 2);
        const float dsc = rd_f16(blk) * (float)q4k_scale(blk + 4, (int)(j & 7));
        const float dmn = rd_f16(blk + 2) * (float)q4k_min(blk + 4, (int)(j & 7));
        acc += dsc * xd * (float)dot - dmn * xsum;
      }
      out[r * out_features + n] = acc;
    }
}

/* acc += xd*(s0*dot0 + s1*dot1) per 32-group.  xq: 160-byte D4S4 blocks. */
void oracle_q6_k_d4s4_mmq(const uint8_t* xq, const uint8_t* w, float* out,
                          int64_t rows, int64_t in_features, int64_t out_features) {
  const int64_t nsb = in_features / 32, row_bytes = in_features / QK_K * Q6_K_BYTES;
  const int64_t x_row_bytes = in_features / 128 * D4S4_BYTES;
#pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < out_features; ++n)
    for (int64_t r = 0; r < rows; ++r) {
      float acc = 0.0f;
      for (int64_t j = 0; j < nsb; ++j) {
        const uint8_t* blk = w + n * row_bytes + (j >> 3) * Q6_K_BYTES;
        const uint8_t* xb = xq + r * x_row_bytes + (j >> 2) * D4S4_BYTES;
        const int8_t* q8 = (const int8_t*)(xb + 32) + (j & 3) * 32;
        int32_t dot0 = 0, dot1 = 0;
        const int g = (int)(j & 7);
        for (int i = 0; i < 16; ++i) {
          dot0 += q6k_quant(blk, g * 32 + i) * (int32_t)q8[i];
          dot1 += q6k_quant(blk, g * 32 + 16 + i) * (int32_t)q8[16 + i];
        }
        float xd;
        memcpy(&xd, xb + 4 * (j & 3), 4);
        const float d = rd_f16(blk + 208);
        const int8_t* sc = (const int8_t*)(blk + 192);
        acc += xd * (d * (float)sc[2 * g] * (float)dot0 + d * (float)sc[2 * g + 1] * (float)dot1);
      }
      out[r * out_features + n] = acc;
    }
}

int oracle_num_threads(void) {
  int n = 1;
#ifdef _OPENMP
#pragma omp parallel
  {
#pragma omp master
    n = omp_get_num_threads();
  }
#endif
  return n;
}
