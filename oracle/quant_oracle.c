/*
 * CPU oracle for cogni-ml's quantized-matmul hot path.
 *
 * THIS FILE IS TEST INFRASTRUCTURE. It is a plain-C restatement of the
 * reference's Crystal algorithm, used only as the parity checker (tests,
 * the smoke check) and as the timed CPU baseline in the benchmark. The
 * product path (the HIP kernels and the C-ABI library) never links, loads or
 * calls anything in this directory.
 *
 * Source of truth (reference, Crystal):
 *   src/ml/gguf/dequant.cr        bulk dequantize, get_scale_min_k4, fp16_to_f32
 *   src/ml/gguf/quant_matmul.cr   fused dequant + matmul with Float64 accumulation
 *   src/ml/gguf/reader.cr:34-127  TensorType geometry, TensorInfo#data_bytes
 *
 * Crystal arithmetic rules this restatement relies on:
 *   Float32 * Float32 -> Float32            Float32 * Int / UInt8 -> Float32
 *   Float64 * Float32 -> Float64            Float32 * Float64 -> Float64
 *   UInt8 + Int32 -> UInt8 (no overflow on this path, q <= 31)
 *   '*' is left associative; no fast-math; no fused multiply-add contraction.
 * The one assumption that cannot be verified without a Crystal compiler is the
 * last one (LLVM emits separate fmul/fsub for `d1 * q - m1`). It is the
 * two-rounding reading, which is also what the reference's own comparison
 * against ggml (spec/q4k_dequant_spec.cr:71-73) presumes.
 *
 * Build: gcc -O2 -ffp-contract=off (see oracle/Makefile). Every statement that
 * must round separately is written as its own assignment to a typed variable.
 *
 * Pinning status (see tests/test_oracle_*.py): every function below is pinned
 * by at least one check that does not restate its own formula: an exhaustive
 * 65 536-input sweep against IEEE binary16 (numpy), the reference's own
 * IQ4_NL known-answer vectors (spec/iq4_nl_dequant_spec.cr:34-106), inverse
 * packing brute force for the 6-bit scale fields, closed-form blocks,
 * element-order blocks, an independent vectorised numpy restatement written
 * from the block-layout comments, and the fused == bulk-dequant + f64 dot
 * invariant the reference tests in spec/q4k_matmul_spec.cr:15-34,85-88.
 */
#include <stdint.h>
#include <string.h>
#include <math.h>

#define QK_K 256
#define QK4_NL 32

/* ggml tensor type ids, reader.cr:34-49 */
enum {
  TT_F32 = 0, TT_F16 = 1, TT_Q4_0 = 2, TT_Q4_1 = 3, TT_Q5_0 = 6, TT_Q5_1 = 7,
  TT_Q8_0 = 8, TT_Q2_K = 10, TT_Q3_K = 11, TT_Q4_K = 12, TT_Q5_K = 13,
  TT_Q6_K = 14, TT_Q8_K = 15, TT_IQ4_NL = 20
};

/* reader.cr:51-68. Returns -1 for an id that is not in the enum. */
int oracle_block_bytes(uint32_t type) {
  switch (type) {
    case TT_F32: return 4;   case TT_F16: return 2;
    case TT_Q4_0: return 18; case TT_Q4_1: return 20;
    case TT_Q5_0: return 22; case TT_Q5_1: return 24;
    case TT_Q8_0: return 34; case TT_Q2_K: return 84;
    case TT_Q3_K: return 110; case TT_Q4_K: return 144;
    case TT_Q5_K: return 176; case TT_Q6_K: return 210;
    case TT_Q8_K: return 292; case TT_IQ4_NL: return 18;
    default: return -1;
  }
}

/* reader.cr:71-78 */
int oracle_block_elements(uint32_t type) {
  switch (type) {
    case TT_F32: case TT_F16: return 1;
    case TT_Q4_0: case TT_Q4_1: case TT_Q5_0: case TT_Q5_1: case TT_Q8_0: return 32;
    case TT_Q2_K: case TT_Q3_K: case TT_Q4_K: case TT_Q5_K: case TT_Q6_K: case TT_Q8_K: return 256;
    case TT_IQ4_NL: return 32;
    default: return -1;
  }
}

/* TensorInfo#data_bytes, reader.cr:119-127 */
int64_t oracle_data_bytes(uint32_t type, int64_t n_elements) {
  int bb = oracle_block_bytes(type), be = oracle_block_elements(type);
  if (bb < 0) return -1;
  if (type == TT_F32 || type == TT_F16) return n_elements * bb;
  return ((n_elements + be - 1) / be) * bb;
}

/* dequant.cr:257-283. Software binary16 -> binary32; NaN loses sign and payload. */
float oracle_fp16_to_f32(uint16_t h) {
  uint32_t sign = (h >> 15) & 1u;
  uint32_t expo = (h >> 10) & 0x1Fu;
  uint32_t mant = h & 0x03FFu;
  float f;
  if (expo == 0) {
    if (mant == 0) return sign ? -0.0f : 0.0f;
    f = (float)mant / 1024.0f;
    f = f * ldexpf(1.0f, -14);
    return sign ? -f : f;
  } else if (expo == 31) {
    if (mant == 0) return sign ? -INFINITY : INFINITY;
    { uint32_t bits = 0x7FC00000u; float r; memcpy(&r, &bits, 4); return r; }
  }
  {
    float frac = (float)mant / 1024.0f;
    float one_plus = 1.0f + frac;
    f = one_plus * ldexpf(1.0f, (int)expo - 15);
  }
  return sign ? -f : f;
}

static inline float rd_f16(const uint8_t *p) { /* dequant.cr:252-255, little endian */
  return oracle_fp16_to_f32((uint16_t)(p[0] | ((uint16_t)p[1] << 8)));
}

/* dequant.cr:240-249 */
void oracle_get_scale_min_k4(int j, const uint8_t *scales, float *sc, float *m) {
  if (j < 4) {
    *sc = (float)(scales[j] & 63);
    *m = (float)(scales[j + 4] & 63);
  } else {
    *sc = (float)(uint8_t)((scales[j + 4] & 0x0F) | ((scales[j - 4] >> 6) << 4));
    *m = (float)(uint8_t)((scales[j + 4] >> 4) | ((scales[j] >> 6) << 4));
  }
}

/* dequant.cr:11-16 */
static const int8_t IQ4_NL_VALUES[16] = {
  -127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};

/* dequant.cr:34-40 */
void oracle_dequantize_f32(const uint8_t *data, int n, float *out) {
  for (int i = 0; i < n; i++) memcpy(&out[i], data + (size_t)i * 4, 4);
}

/* dequant.cr:43-49 */
void oracle_dequantize_f16(const uint8_t *data, int n, float *out) {
  for (int i = 0; i < n; i++) out[i] = rd_f16(data + (size_t)i * 2);
}

/* dequant.cr:53-71 */
void oracle_dequantize_q8_0(const uint8_t *data, int n, float *out) {
  int nb = (n + 31) / 32;
  for (int i = 0; i < n; i++) out[i] = 0.0f;
  for (int i = 0; i < nb; i++) {
    const uint8_t *blk = data + (size_t)i * 34;
    float d = rd_f16(blk);
    const int8_t *qs = (const int8_t *)(blk + 2);
    int base = i * 32;
    int count = n - base < 32 ? n - base : 32;
    for (int j = 0; j < count; j++) {
      float q = (float)qs[j];
      out[base + j] = d * q;
    }
  }
}

/* dequant.cr:76-101 */
void oracle_dequantize_iq4_nl(const uint8_t *data, int n, float *out) {
  int nb = (n + QK4_NL - 1) / QK4_NL;
  for (int i = 0; i < n; i++) out[i] = 0.0f;
  for (int i = 0; i < nb; i++) {
    const uint8_t *blk = data + (size_t)i * 18;
    float d = rd_f16(blk);
    const uint8_t *qs = blk + 2;
    int base = i * QK4_NL;
    int first = n - base < 16 ? n - base : 16;
    for (int j = 0; j < first; j++) out[base + j] = d * (float)IQ4_NL_VALUES[qs[j] & 0x0F];
    int sbase = base + 16;
    int second = n - sbase < 16 ? n - sbase : 16;
    for (int j = 0; j < second; j++) out[sbase + j] = d * (float)IQ4_NL_VALUES[qs[j] >> 4];
  }
}

/* dequant.cr:106-142 */
void oracle_dequantize_q4_k(const uint8_t *data, int n, float *out) {
  int nb = n / QK_K;
  for (int i = 0; i < n; i++) out[i] = 0.0f;
  for (int i = 0; i < nb; i++) {
    const uint8_t *blk = data + (size_t)i * 144;
    float d = rd_f16(blk);
    float dmin = rd_f16(blk + 2);
    const uint8_t *scales = blk + 4;
    const uint8_t *qs = blk + 16;
    int is = 0;
    int yi = i * QK_K;
    for (int g = 0; g < 4; g++) {
      float sc, m, sc2, m2;
      oracle_get_scale_min_k4(is, scales, &sc, &m);
      float d1 = d * sc;
      float m1 = dmin * m;
      oracle_get_scale_min_k4(is + 1, scales, &sc2, &m2);
      float d2 = d * sc2;
      float m2f = dmin * m2;
      for (int l = 0; l < 32; l++) {
        float prod = d1 * (float)(qs[l] & 0x0F);
        out[yi + l] = prod - m1;
      }
      for (int l = 0; l < 32; l++) {
        float prod = d2 * (float)(qs[l] >> 4);
        out[yi + 32 + l] = prod - m2f;
      }
      qs += 32; is += 2; yi += 64;
    }
  }
}

/* dequant.cr:146-193 */
void oracle_dequantize_q5_k(const uint8_t *data, int n, float *out) {
  int nb = n / QK_K;
  int yi = 0;
  for (int i = 0; i < n; i++) out[i] = 0.0f;
  for (int i = 0; i < nb; i++) {
    const uint8_t *blk = data + (size_t)i * 176;
    float d = rd_f16(blk);
    float dmin = rd_f16(blk + 2);
    const uint8_t *scales = blk + 4;
    const uint8_t *qh = blk + 16;
    const uint8_t *ql = blk + 48;
    uint8_t u1 = 1, u2 = 2;
    int is = 0;
    for (int g = 0; g < 4; g++) {
      float sc, m, sc2, m2v;
      oracle_get_scale_min_k4(is, scales, &sc, &m);
      float d1 = d * sc;
      float m1 = dmin * m;
      oracle_get_scale_min_k4(is + 1, scales, &sc2, &m2v);
      float d2 = d * sc2;
      float m2 = dmin * m2v;
      for (int l = 0; l < 32; l++) {
        uint8_t q = (uint8_t)((ql[l] & 0x0F) + ((qh[l] & u1) ? 16 : 0));
        float prod = d1 * (float)q;
        out[yi++] = prod - m1;
      }
      for (int l = 0; l < 32; l++) {
        uint8_t q = (uint8_t)(((ql[l] >> 4) & 0x0F) + ((qh[l] & u2) ? 16 : 0));
        float prod = d2 * (float)q;
        out[yi++] = prod - m2;
      }
      ql += 32; is += 2;
      u1 = (uint8_t)(u1 << 2); u2 = (uint8_t)(u2 << 2);
    }
  }
}

/* dequant.cr:197-236 */
void oracle_dequantize_q6_k(const uint8_t *data, int n, float *out) {
  int nb = n / QK_K;
  int yi = 0;
  for (int i = 0; i < n; i++) out[i] = 0.0f;
  for (int i = 0; i < nb; i++) {
    const uint8_t *blk = data + (size_t)i * 210;
    const uint8_t *ql = blk;
    const uint8_t *qh = blk + 128;
    const int8_t *sc = (const int8_t *)(blk + 192);
    float d = rd_f16(blk + 208);
    for (int half = 0; half < 2; half++) {
      for (int l = 0; l < 32; l++) {
        int is = l / 16;
        int q1 = ((ql[l] & 0xF) | (((qh[l] >> 0) & 3) << 4)) - 32;
        int q2 = ((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32;
        int q3 = ((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
        int q4 = ((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
        float s0 = d * (float)sc[is];
        float s2 = d * (float)sc[is + 2];
        float s4 = d * (float)sc[is + 4];
        float s6 = d * (float)sc[is + 6];
        out[yi + l] = s0 * (float)q1;
        out[yi + l + 32] = s2 * (float)q2;
        out[yi + l + 64] = s4 * (float)q3;
        out[yi + l + 96] = s6 * (float)q4;
      }
      yi += 128; ql += 64; qh += 32; sc += 8;
    }
  }
}

/* dequant.cr:19-31. Returns 0, or -1 for "Unsupported dequantization type". */
int oracle_dequantize(const uint8_t *data, uint32_t type, int n, float *out) {
  switch (type) {
    case TT_F32: oracle_dequantize_f32(data, n, out); return 0;
    case TT_F16: oracle_dequantize_f16(data, n, out); return 0;
    case TT_Q4_K: oracle_dequantize_q4_k(data, n, out); return 0;
    case TT_Q5_K: oracle_dequantize_q5_k(data, n, out); return 0;
    case TT_Q6_K: oracle_dequantize_q6_k(data, n, out); return 0;
    case TT_Q8_0: oracle_dequantize_q8_0(data, n, out); return 0;
    case TT_IQ4_NL: oracle_dequantize_iq4_nl(data, n, out); return 0;
    default: return -1;
  }
}

/* ---- fused matmul, quant_matmul.cr ------------------------------------- */
/* Every kernel computes result[r*out_dim + o] for o in [o_begin, o_end) so the
 * benchmark can split output rows across host threads; the reference's single
 * thread is o_begin = 0, o_end = out_dim. */

/* quant_matmul.cr:41-99 */
static void mm_q4k(const float *x, int rows, int in_dim, const uint8_t *w, int out_dim,
                   const float *bias, float *result, int o_begin, int o_end) {
  int nb = in_dim / QK_K;
  size_t row_bytes = (size_t)nb * 144;
  for (int r = 0; r < rows; r++) {
    const float *xr = x + (size_t)r * in_dim;
    for (int o = o_begin; o < o_end; o++) {
      double sum = (double)bias[o];
      const uint8_t *w_row = w + (size_t)o * row_bytes;
      for (int blk = 0; blk < nb; blk++) {
        const uint8_t *bp = w_row + (size_t)blk * 144;
        double d = (double)rd_f16(bp);
        double dmin = (double)rd_f16(bp + 2);
        const uint8_t *scales = bp + 4;
        const uint8_t *qs = bp + 16;
        int base_j = blk * QK_K;
        int is = 0, qs_off = 0;
        for (int g = 0; g < 4; g++) {
          float sc, m, sc2, m2;
          oracle_get_scale_min_k4(is, scales, &sc, &m);
          double d1 = d * (double)sc, m1 = dmin * (double)m;
          oracle_get_scale_min_k4(is + 1, scales, &sc2, &m2);
          double d2 = d * (double)sc2, m2v = dmin * (double)m2;
          for (int l = 0; l < 32; l++) {
            int j = base_j + (is / 2) * 64 + l;
            int q = qs[qs_off + l] & 0x0F;
            double val = d1 * (double)q - m1;
            sum += (double)xr[j] * val;
          }
          for (int l = 0; l < 32; l++) {
            int j = base_j + (is / 2) * 64 + 32 + l;
            int q = qs[qs_off + l] >> 4;
            double val = d2 * (double)q - m2v;
            sum += (double)xr[j] * val;
          }
          qs_off += 32; is += 2;
        }
      }
      result[(size_t)r * out_dim + o] = (float)sum;
    }
  }
}

/* quant_matmul.cr:103-168 */
static void mm_q5k(const float *x, int rows, int in_dim, const uint8_t *w, int out_dim,
                   const float *bias, float *result, int o_begin, int o_end) {
  int nb = in_dim / QK_K;
  size_t row_bytes = (size_t)nb * 176;
  for (int r = 0; r < rows; r++) {
    const float *xr = x + (size_t)r * in_dim;
    for (int o = o_begin; o < o_end; o++) {
      double sum = (double)bias[o];
      const uint8_t *w_row = w + (size_t)o * row_bytes;
      for (int blk = 0; blk < nb; blk++) {
        const uint8_t *bp = w_row + (size_t)blk * 176;
        double d = (double)rd_f16(bp);
        double dmin = (double)rd_f16(bp + 2);
        const uint8_t *scales = bp + 4;
        const uint8_t *qh = bp + 16;
        const uint8_t *ql = bp + 48;
        int base_j = blk * QK_K;
        uint8_t u1 = 1, u2 = 2;
        int is = 0, ql_off = 0;
        for (int g = 0; g < 4; g++) {
          float sc, m, sc2, m2;
          oracle_get_scale_min_k4(is, scales, &sc, &m);
          double d1 = d * (double)sc, m1 = dmin * (double)m;
          oracle_get_scale_min_k4(is + 1, scales, &sc2, &m2);
          double d2 = d * (double)sc2, m2v = dmin * (double)m2;
          for (int l = 0; l < 32; l++) {
            int j = base_j + (is / 2) * 64 + l;
            uint8_t q = (uint8_t)((ql[ql_off + l] & 0x0F) + ((qh[l] & u1) ? 16 : 0));
            double val = d1 * (double)q - m1;
            sum += (double)xr[j] * val;
          }
          for (int l = 0; l < 32; l++) {
            int j = base_j + (is / 2) * 64 + 32 + l;
            uint8_t q = (uint8_t)(((ql[ql_off + l] >> 4) & 0x0F) + ((qh[l] & u2) ? 16 : 0));
            double val = d2 * (double)q - m2v;
            sum += (double)xr[j] * val;
          }
          ql_off += 32; is += 2;
          u1 = (uint8_t)(u1 << 2); u2 = (uint8_t)(u2 << 2);
        }
      }
      result[(size_t)r * out_dim + o] = (float)sum;
    }
  }
}

/* quant_matmul.cr:171-231. Summation order per l is l, l+32, l+64, l+96. */
static void mm_q6k(const float *x, int rows, int in_dim, const uint8_t *w, int out_dim,
                   const float *bias, float *result, int o_begin, int o_end) {
  int nb = in_dim / QK_K;
  size_t row_bytes = (size_t)nb * 210;
  for (int r = 0; r < rows; r++) {
    const float *xr = x + (size_t)r * in_dim;
    for (int o = o_begin; o < o_end; o++) {
      double sum = (double)bias[o];
      const uint8_t *w_row = w + (size_t)o * row_bytes;
      for (int blk = 0; blk < nb; blk++) {
        const uint8_t *bp = w_row + (size_t)blk * 210;
        const uint8_t *ql = bp;
        const uint8_t *qh = bp + 128;
        const int8_t *sc = (const int8_t *)(bp + 192);
        double d = (double)rd_f16(bp + 208);
        int base_j = blk * QK_K;
        for (int half = 0; half < 2; half++) {
          for (int l = 0; l < 32; l++) {
            int is = l / 16;
            int q1 = ((ql[l] & 0xF) | (((qh[l] >> 0) & 3) << 4)) - 32;
            int q2 = ((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32;
            int q3 = ((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
            int q4 = ((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
            double s0 = (double)sc[is], s2 = (double)sc[is + 2];
            double s4 = (double)sc[is + 4], s6 = (double)sc[is + 6];
            int jb = base_j + half * 128;
            sum += (double)xr[jb + l] * (d * s0 * (double)q1);
            sum += (double)xr[jb + l + 32] * (d * s2 * (double)q2);
            sum += (double)xr[jb + l + 64] * (d * s4 * (double)q3);
            sum += (double)xr[jb + l + 96] * (d * s6 * (double)q4);
          }
          ql += 64; qh += 32; sc += 8;
        }
      }
      result[(size_t)r * out_dim + o] = (float)sum;
    }
  }
}

/* quant_matmul.cr:235-270 */
static void mm_q8_0(const float *x, int rows, int in_dim, const uint8_t *w, int out_dim,
                    const float *bias, float *result, int o_begin, int o_end) {
  int nb = (in_dim + 31) / 32;
  size_t row_bytes = (size_t)nb * 34;
  for (int r = 0; r < rows; r++) {
    const float *xr = x + (size_t)r * in_dim;
    for (int o = o_begin; o < o_end; o++) {
      double sum = (double)bias[o];
      const uint8_t *w_row = w + (size_t)o * row_bytes;
      for (int blk = 0; blk < nb; blk++) {
        const uint8_t *bp = w_row + (size_t)blk * 34;
        double d = (double)rd_f16(bp);
        const int8_t *qs = (const int8_t *)(bp + 2);
        int base_j = blk * 32;
        int count = in_dim - base_j < 32 ? in_dim - base_j : 32;
        for (int j = 0; j < count; j++) sum += (double)xr[base_j + j] * (d * (double)qs[j]);
      }
      result[(size_t)r * out_dim + o] = (float)sum;
    }
  }
}

/* quant_matmul.cr:274-323 */
static void mm_iq4_nl(const float *x, int rows, int in_dim, const uint8_t *w, int out_dim,
                      const float *bias, float *result, int o_begin, int o_end) {
  int nb = (in_dim + QK4_NL - 1) / QK4_NL;
  size_t row_bytes = (size_t)nb * 18;
  for (int r = 0; r < rows; r++) {
    const float *xr = x + (size_t)r * in_dim;
    for (int o = o_begin; o < o_end; o++) {
      double sum = (double)bias[o];
      const uint8_t *w_row = w + (size_t)o * row_bytes;
      for (int blk = 0; blk < nb; blk++) {
        const uint8_t *bp = w_row + (size_t)blk * 18;
        double d = (double)rd_f16(bp);
        const uint8_t *qs = bp + 2;
        int base_j = blk * QK4_NL;
        int first = in_dim - base_j < 16 ? in_dim - base_j : 16;
        for (int j = 0; j < first; j++) {
          double val = d * (double)IQ4_NL_VALUES[qs[j] & 0x0F];
          sum += (double)xr[base_j + j] * val;
        }
        int sbase = base_j + 16;
        int second = in_dim - sbase < 16 ? in_dim - sbase : 16;
        for (int j = 0; j < second; j++) {
          double val = d * (double)IQ4_NL_VALUES[qs[j] >> 4];
          sum += (double)xr[sbase + j] * val;
        }
      }
      result[(size_t)r * out_dim + o] = (float)sum;
    }
  }
}

/* quant_matmul.cr:326-345. x * w is a Float32 product, widened when added. */
static void mm_f32(const float *x, int rows, int in_dim, const uint8_t *w, int out_dim,
                   const float *bias, float *result, int o_begin, int o_end) {
  for (int r = 0; r < rows; r++) {
    const float *xr = x + (size_t)r * in_dim;
    for (int o = o_begin; o < o_end; o++) {
      double sum = (double)bias[o];
      const uint8_t *w_row = w + (size_t)o * in_dim * 4;
      for (int j = 0; j < in_dim; j++) {
        float wv; memcpy(&wv, w_row + (size_t)j * 4, 4);
        float prod = xr[j] * wv;
        sum += (double)prod;
      }
      result[(size_t)r * out_dim + o] = (float)sum;
    }
  }
}

/* quant_matmul.cr:348-368. Same Float32 product as the F32 case. */
static void mm_f16(const float *x, int rows, int in_dim, const uint8_t *w, int out_dim,
                   const float *bias, float *result, int o_begin, int o_end) {
  for (int r = 0; r < rows; r++) {
    const float *xr = x + (size_t)r * in_dim;
    for (int o = o_begin; o < o_end; o++) {
      double sum = (double)bias[o];
      const uint8_t *w_row = w + (size_t)o * in_dim * 2;
      for (int j = 0; j < in_dim; j++) {
        float val = rd_f16(w_row + (size_t)j * 2);
        float prod = xr[j] * val;
        sum += (double)prod;
      }
      result[(size_t)r * out_dim + o] = (float)sum;
    }
  }
}

/* quant_matmul.cr:20-36 restricted to output rows [o_begin, o_end).
 * Returns 0, or -1 for "Unsupported quant type for fused matmul". */
int oracle_matmul_add_range(const float *x, int rows, int in_dim, const uint8_t *w_raw,
                            uint32_t w_type, int out_dim, const float *bias, float *result,
                            int o_begin, int o_end) {
  switch (w_type) {
    case TT_Q4_K: mm_q4k(x, rows, in_dim, w_raw, out_dim, bias, result, o_begin, o_end); return 0;
    case TT_Q5_K: mm_q5k(x, rows, in_dim, w_raw, out_dim, bias, result, o_begin, o_end); return 0;
    case TT_Q6_K: mm_q6k(x, rows, in_dim, w_raw, out_dim, bias, result, o_begin, o_end); return 0;
    case TT_Q8_0: mm_q8_0(x, rows, in_dim, w_raw, out_dim, bias, result, o_begin, o_end); return 0;
    case TT_IQ4_NL: mm_iq4_nl(x, rows, in_dim, w_raw, out_dim, bias, result, o_begin, o_end); return 0;
    case TT_F32: mm_f32(x, rows, in_dim, w_raw, out_dim, bias, result, o_begin, o_end); return 0;
    case TT_F16: mm_f16(x, rows, in_dim, w_raw, out_dim, bias, result, o_begin, o_end); return 0;
    default: return -1;
  }
}

/* quant_matmul.cr:20-36, the reference's single-thread form. */
int oracle_matmul_add(const float *x, int rows, int in_dim, const uint8_t *w_raw, uint32_t w_type,
                      int out_dim, const float *bias, float *result) {
  return oracle_matmul_add_range(x, rows, in_dim, w_raw, w_type, out_dim, bias, result, 0, out_dim);
}

/* The CPU check of the reference's SwiGLU probe (bin/cuda_ffn_sequence_probe.cr:189-191 and its use on
 * gate/up): silu(g) = g / (1 + exp(-g)) in Float32 (Math.exp on a Float32 is the single-precision libm exp),
 * then silu(g) * u in Float32. Pinned by the closed forms silu(0) = 0, silu(x) - silu(-x) = x and a float64
 * evaluation (tests/test_oracle_matmul.py). */
void oracle_swiglu(const float *gate, const float *up, float *out, int64_t n) {
  for (int64_t i = 0; i < n; i++) {
    const float g = gate[i];
    const float e = expf(-g);
    const float den = 1.0f + e;
    const float s = g / den;
    out[i] = s * up[i];
  }
}

/* RMSNorm of one dim-length vector as src/ml/gguf/qwen35_cpu.cr:484-490: the sum of squares in Float64 over
 * x widened element by element, inv_rms = (1 / sqrt(ss / dim + eps)) rounded to Float32, then x[j] * inv_rms * w[j]
 * left to right in Float32. Pinned by closed forms (constant vectors, unit weights: mean square of the output is
 * ms / (ms + eps)), scale invariance at eps = 0 and a float64 numpy evaluation (tests/test_oracle_matmul.py). */
void oracle_rms_norm(const float *x, const float *w, float *out, int64_t dim, float eps) {
  double ss = 0.0;
  for (int64_t j = 0; j < dim; j++) ss += (double)x[j] * (double)x[j];
  const float inv_rms = (float)(1.0 / sqrt(ss / (double)dim + (double)eps));
  for (int64_t j = 0; j < dim; j++) {
    const float t = x[j] * inv_rms;
    out[j] = t * w[j];
  }
}
