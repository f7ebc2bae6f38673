/* Scalar C restatement of the reference's quantized-weight linear path.  TEST INFRASTRUCTURE ONLY: the checker and the
 * timed CPU baseline; never linked into the shipped library.
 *
 * Dequant loops restate the published ggml reference routines (ggml-quants.c dequantize_row_q4_0 / q8_0 / q4_K / q5_K /
 * q6_K / mxfp4; gguf-py >= 0.18 is what the reference's tests call, pyproject.toml:79) element by element, independently of
 * the vectorised numpy restatement of tinygrad/llm/gguf.py:46,56,68-72,105-114 in oracle/ggml.py: the two must agree
 * bit for bit (tests/test_oracle_ggml.py).
 * The linear restates Tensor.dot (tinygrad/mixin/op.py:367-392) with sum_acc_dtype = float32 (tinygrad/dtype.py:212-216).
 */
#include <stdint.h>
#include <string.h>
#include <math.h>
#include <stdlib.h>
#include <immintrin.h>
#ifdef _OPENMP
#include <omp.h>
#endif

static inline float h2f(uint16_t h) {
  uint32_t s = (uint32_t)(h & 0x8000u) << 16, e = (h >> 10) & 0x1f, m = h & 0x3ffu, u;
  if (e == 0) {
    if (m == 0) u = s;
    else { int sh = 0; while (!(m & 0x400u)) { m <<= 1; sh++; } m &= 0x3ffu; u = s | ((uint32_t)(113 - sh) << 23) | (m << 13); }
  } else if (e == 31) u = s | 0x7f800000u | (m << 13);
  else u = s | ((e + 112) << 23) | (m << 13);
  float f; memcpy(&f, &u, 4); return f;
}
/* round-to-nearest-even float32 -> float16 bits (the cast at tinygrad/llm/model.py:376) */
static inline uint16_t f2h(float f) {
  uint32_t x; memcpy(&x, &f, 4);
  uint32_t s = (x >> 16) & 0x8000u, a = x & 0x7fffffffu;
  if (a >= 0x7f800000u) return (uint16_t)(s | 0x7c00u | ((a > 0x7f800000u) ? 0x200u : 0));
  if (a >= 0x477ff000u) return (uint16_t)(s | 0x7c00u);           /* >= 65520 rounds to inf */
  if (a < 0x33000001u) return (uint16_t)s;                         /* <= 2^-25 rounds to zero */
  int e = (int)(a >> 23) - 127;
  uint32_t m = (a & 0x7fffffu) | 0x800000u;
  int shift = (e < -14) ? (13 + (-14 - e)) : 13;
  uint32_t r = m >> shift, rem = m & ((1u << shift) - 1), half = 1u << (shift - 1);
  if (rem > half || (rem == half && (r & 1))) r++;
  if (e < -14) return (uint16_t)(s | r);                           /* subnormal (r may carry into exponent 1: fine) */
  return (uint16_t)(s | (((uint32_t)(e + 15) << 10) + (r - 0x400u)));
}
/* x[i] = float32(float16(x[i])), round-to-nearest-even, n a multiple of 8: the F16C conversions (part of the x86-64-v3 baseline this file is built for), which
 * tests/test_oracle_ggml.py holds against the bit-level f2h / h2f above.  The per-weight software round trip was most of orc_linear's time. */
static inline void round_f16_block(float* x, int n) {
  for (int j = 0; j < n; j += 8) _mm256_storeu_ps(x + j, _mm256_cvtph_ps(_mm256_cvtps_ph(_mm256_loadu_ps(x + j), _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC)));
}
void orc_round_f16(float* x, int64_t n) { for (int64_t j = 0; j + 8 <= n; j += 8) round_f16_block(x + j, 8); for (int64_t j = n & ~(int64_t)7; j < n; j++) x[j] = h2f(f2h(x[j])); }
float orc_h2f(uint16_t h) { return h2f(h); }
uint16_t orc_f2h(float f) { return f2h(f); }

/* ---- block dequant: y gets nb * nel floats ---- */
static void deq_q4_0(const uint8_t* b, float* y) {            /* block_q4_0: ggml_common.py:21 */
  uint16_t dh; memcpy(&dh, b, 2); const float d = h2f(dh);
  for (int j = 0; j < 16; j++) {
    y[j]      = (float)((int)(b[2 + j] & 0x0F) - 8) * d;
    y[j + 16] = (float)((int)(b[2 + j] >> 4) - 8) * d;
  }
}
static void deq_q8_0(const uint8_t* b, float* y) {            /* block_q8_0: ggml_common.py:59-64 */
  uint16_t dh; memcpy(&dh, b, 2); const float d = h2f(dh);
  for (int j = 0; j < 32; j++) y[j] = (float)(int8_t)b[2 + j] * d;
}
static void deq_q6_k(const uint8_t* b, float* y) {            /* block_q6_K: ggml_common.py:123-129 */
  uint16_t dh; memcpy(&dh, b + 208, 2); const float d = h2f(dh);
  const uint8_t *ql = b, *qh = b + 128; const int8_t* sc = (const int8_t*)(b + 192);
  for (int n = 0; n < 256; n += 128) {
    for (int l = 0; l < 32; l++) {
      int is = l / 16;
      int q1 = (int)((ql[l]      & 0xF) | (((qh[l] >> 0) & 3) << 4)) - 32;
      int q2 = (int)((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32;
      int q3 = (int)((ql[l]      >> 4)  | (((qh[l] >> 4) & 3) << 4)) - 32;
      int q4 = (int)((ql[l + 32] >> 4)  | (((qh[l] >> 6) & 3) << 4)) - 32;
      y[l]      = d * sc[is + 0] * q1;
      y[l + 32] = d * sc[is + 2] * q2;
      y[l + 64] = d * sc[is + 4] * q3;
      y[l + 96] = d * sc[is + 6] * q4;
    }
    y += 128; ql += 64; qh += 32; sc += 8;
  }
}
/* block_q4_1: d, m, qs[16]  (dequantize_row_q4_1; tinygrad/llm/gguf.py:47-49) */
static void deq_q4_1(const uint8_t* b, float* y) {
  uint16_t dh, mh; memcpy(&dh, b, 2); memcpy(&mh, b + 2, 2);
  const float d = h2f(dh), m = h2f(mh);
  for (int j = 0; j < 16; j++) { y[j] = (float)(b[4 + j] & 0x0F) * d + m; y[j + 16] = (float)(b[4 + j] >> 4) * d + m; }
}
/* block_q5_0: d, qh[4], qs[16] and block_q5_1: d, m, qh[4], qs[16]  (dequantize_row_q5_0 / q5_1; tinygrad/llm/gguf.py:50-55).
 * ggml evaluates Q5_0 as (q - 16) * d; the reference evaluates q * d + (-16 * d).  Both are exact for finite d (5 x 11 significant
 * bits), they differ for an infinite d, and bit-exactness is owed to the reference, so its form is the one used here. */
static void deq_q5(const uint8_t* b, float* y, int one) {
  uint16_t dh, mh = 0; memcpy(&dh, b, 2); if (one) memcpy(&mh, b + 2, 2);
  const float d = h2f(dh), off = one ? h2f(mh) : -16.0f * d;
  const uint8_t* p = b + (one ? 4 : 2);
  uint32_t qh; memcpy(&qh, p, 4);
  for (int j = 0; j < 16; j++) {
    const int x0 = (p[4 + j] & 0x0F) | (int)(((qh >> j) & 1u) << 4), x1 = (p[4 + j] >> 4) | (int)(((qh >> (j + 16)) & 1u) << 4);
    y[j] = (float)x0 * d + off; y[j + 16] = (float)x1 * d + off;
  }
}
/* block_iq4_xs: d, scales_h, scales_l[4], qs[128]  (dequantize_row_iq4_xs; tinygrad/llm/gguf.py:96-104) */
static const int8_t kvalues_iq4nl[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};
static void deq_iq4_xs(const uint8_t* b, float* y) {
  uint16_t dh, sh; memcpy(&dh, b, 2); memcpy(&sh, b + 2, 2);
  const float d = h2f(dh);
  const uint8_t* qs = b + 8;
  for (int ib = 0; ib < 8; ib++) {
    const int ls = ((b[4 + ib / 2] >> (4 * (ib % 2))) & 0xf) | (((sh >> (2 * ib)) & 3) << 4);
    const float dl = d * (float)(ls - 32);
    for (int j = 0; j < 16; j++) { y[j] = dl * kvalues_iq4nl[qs[j] & 0xf]; y[j + 16] = dl * kvalues_iq4nl[qs[j] >> 4]; }
    y += 32; qs += 16;
  }
}
/* The codebook types.  An entry of a codebook is kept as its digits over the codebook's alphabet (iq_grids.h). */
#include "iq_grids.h"
static int iq3xxs_value(int idx, int j) { const int dg = (IQ3XXS_CODE[idx] >> (3 * j)) & 7; return dg == 7 ? 62 : 4 + 8 * dg; }
static int iq3s_value(int idx, int j) { return 1 + 2 * ((IQ3S_CODE[idx] >> (3 * j)) & 7); }
static int iq2s_value(int idx, int j) { int c = IQ2S_CODE[idx]; for (int i = 0; i < j; i++) c /= 3; static const int a[3] = {8, 25, 43}; return a[c % 3]; }
/* block_iq3_xxs: d, qs[64] indices, 8 x uint32 {4 x 7-bit sign index, 4-bit scale}  (dequantize_row_iq3_xxs; tinygrad/llm/gguf.py:73-81) */
static void deq_iq3_xxs(const uint8_t* b, float* y) {
  uint16_t dh; memcpy(&dh, b, 2);
  const float d = h2f(dh);
  const uint8_t* qs = b + 2;
  for (int ib = 0; ib < 8; ib++) {
    uint32_t aux; memcpy(&aux, b + 66 + 4 * ib, 4);
    const float db = d * (0.5f + (float)(aux >> 28)) * 0.5f;
    for (int l = 0; l < 4; l++) {
      const uint32_t s7 = (aux >> (7 * l)) & 127;
      const uint32_t signs = s7 | ((__builtin_popcount(s7) & 1) << 7);     /* ksigns_iq2xs: the eighth bit makes the parity even */
      for (int j = 0; j < 4; j++) {
        y[j]     = db * (float)iq3xxs_value(qs[2 * l], j)     * ((signs >> j) & 1 ? -1.0f : 1.0f);
        y[j + 4] = db * (float)iq3xxs_value(qs[2 * l + 1], j) * ((signs >> (j + 4)) & 1 ? -1.0f : 1.0f);
      }
      y += 8;
    }
    qs += 8;
  }
}
/* block_iq3_s: d, qs[64], qh[8], signs[32], scales[4]  (dequantize_row_iq3_s; tinygrad/llm/gguf.py:82-88) */
static void deq_iq3_s(const uint8_t* b, float* y) {
  uint16_t dh; memcpy(&dh, b, 2);
  const float d = h2f(dh);
  const uint8_t *qs = b + 2, *qh = b + 66, *sg = b + 74, *sc = b + 106;
  for (int ib = 0; ib < 8; ib++) {
    const float db = d * (float)(1 + 2 * ((sc[ib / 2] >> (4 * (ib % 2))) & 0xf));
    for (int l = 0; l < 4; l++) {
      const int i0 = qs[2 * l] | (((qh[ib] >> (2 * l)) & 1) << 8), i1 = qs[2 * l + 1] | (((qh[ib] >> (2 * l + 1)) & 1) << 8);
      for (int j = 0; j < 4; j++) {
        y[j]     = db * (float)iq3s_value(i0, j) * ((sg[l] >> j) & 1 ? -1.0f : 1.0f);
        y[j + 4] = db * (float)iq3s_value(i1, j) * ((sg[l] >> (j + 4)) & 1 ? -1.0f : 1.0f);
      }
      y += 8;
    }
    qs += 8; sg += 4;
  }
}
/* block_iq2_s: d, qs[32] indices + 32 sign bytes, qh[8], scales[8]  (dequantize_row_iq2_s; tinygrad/llm/gguf.py:89-95) */
static void deq_iq2_s(const uint8_t* b, float* y) {
  uint16_t dh; memcpy(&dh, b, 2);
  const float d = h2f(dh);
  const uint8_t *qs = b + 2, *sg = b + 34, *qh = b + 66, *sc = b + 74;
  for (int ib = 0; ib < 8; ib++) {
    const float db[2] = {d * (0.5f + (float)(sc[ib] & 0xf)) * 0.25f, d * (0.5f + (float)(sc[ib] >> 4)) * 0.25f};
    for (int l = 0; l < 4; l++) {
      const int idx = qs[l] | (((qh[ib] >> (2 * l)) & 3) << 8);
      for (int j = 0; j < 8; j++) y[j] = db[l / 2] * (float)iq2s_value(idx, j) * ((sg[l] >> j) & 1 ? -1.0f : 1.0f);
      y += 8;
    }
    qs += 4; sg += 4;
  }
}
/* block_q1_0: d, 128 sign bits  (tinygrad/llm/gguf.py:115-118): d * (2 bit - 1) */
static void deq_q1_0(const uint8_t* b, float* y) {
  uint16_t dh; memcpy(&dh, b, 2);
  const float d = h2f(dh);
  for (int e = 0; e < 128; e++) y[e] = d * (float)((int)((b[2 + e / 8] >> (e % 8)) & 1) * 2 - 1);
}
/* get_scale_min_k4 of ggml-quants.c: 6-bit scale and min of sub-block j from the 12 packed bytes */
static void scale_min_k4(int j, const uint8_t* q, uint8_t* d, uint8_t* m) {
  if (j < 4) { *d = q[j] & 63; *m = q[j + 4] & 63; }
  else { *d = (uint8_t)((q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4)); *m = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4)); }
}
static void deq_q4_k(const uint8_t* b, float* y) {            /* block_q4_K: d, dmin, scales[12], qs[128]  (dequantize_row_q4_K) */
  uint16_t dh, mh; memcpy(&dh, b, 2); memcpy(&mh, b + 2, 2);
  const float d = h2f(dh), min = h2f(mh);
  const uint8_t* q = b + 16; int is = 0;
  for (int j = 0; j < 256; j += 64) {
    uint8_t sc, m;
    scale_min_k4(is + 0, b + 4, &sc, &m); const float d1 = d * sc, m1 = min * m;
    scale_min_k4(is + 1, b + 4, &sc, &m); const float d2 = d * sc, m2 = min * m;
    for (int l = 0; l < 32; l++) *y++ = d1 * (q[l] & 0xF) - m1;
    for (int l = 0; l < 32; l++) *y++ = d2 * (q[l] >> 4) - m2;
    q += 32; is += 2;
  }
}
static void deq_q5_k(const uint8_t* b, float* y) {            /* block_q5_K: d, dmin, scales[12], qh[32], qs[128]  (dequantize_row_q5_K) */
  uint16_t dh, mh; memcpy(&dh, b, 2); memcpy(&mh, b + 2, 2);
  const float d = h2f(dh), min = h2f(mh);
  const uint8_t *qh = b + 16, *ql = b + 48; int is = 0; uint8_t u1 = 1, u2 = 2;
  for (int j = 0; j < 256; j += 64) {
    uint8_t sc, m;
    scale_min_k4(is + 0, b + 4, &sc, &m); const float d1 = d * sc, m1 = min * m;
    scale_min_k4(is + 1, b + 4, &sc, &m); const float d2 = d * sc, m2 = min * m;
    for (int l = 0; l < 32; l++) *y++ = d1 * ((ql[l] & 0xF) + (qh[l] & u1 ? 16 : 0)) - m1;
    for (int l = 0; l < 32; l++) *y++ = d2 * ((ql[l] >> 4) + (qh[l] & u2 ? 16 : 0)) - m2;
    ql += 32; is += 2; u1 <<= 2; u2 <<= 2;
  }
}
/* ggml's kvalues_mxfp4 is an int8 table (code 8 -> +0); the reference's float LUT (tinygrad/llm/gguf.py:108-110) holds -0.0
 * for code 8, and bit-exactness is owed to the reference, so the table here is the reference's. */
static const float kvalues_mxfp4[16] = {0.0f, 1.0f, 2.0f, 3.0f, 4.0f, 6.0f, 8.0f, 12.0f, -0.0f, -1.0f, -2.0f, -3.0f, -4.0f, -6.0f, -8.0f, -12.0f};
static void deq_mxfp4(const uint8_t* b, float* y) {           /* block_mxfp4: ggml_common.py:35 */
  /* ggml: d = GGML_E8M0_TO_FP32_HALF(e) = 2^(e-128), built from bits so e = 0, 1 give fp32 subnormals */
  uint32_t e = b[0], bits = (e < 2) ? (0x00200000u << e) : ((e - 1) << 23);
  float d; memcpy(&d, &bits, 4);
  for (int j = 0; j < 16; j++) {
    y[j]      = kvalues_mxfp4[b[1 + j] & 0x0F] * d;
    y[j + 16] = kvalues_mxfp4[b[1 + j] >> 4] * d;
  }
}

static int type_geom(int t, int* nel, int* nby) {
  switch (t) { case 2: *nel = 32; *nby = 18; return 0; case 8: *nel = 32; *nby = 34; return 0;
               case 23: *nel = 256; *nby = 136; return 0; case 41: *nel = 128; *nby = 18; return 0;
               case 18: *nel = 256; *nby = 98; return 0; case 21: *nel = 256; *nby = 110; return 0; case 22: *nel = 256; *nby = 82; return 0;
               case 3: *nel = 32; *nby = 20; return 0; case 6: *nel = 32; *nby = 22; return 0; case 7: *nel = 32; *nby = 24; return 0;
               case 12: *nel = 256; *nby = 144; return 0; case 13: *nel = 256; *nby = 176; return 0;
               case 14: *nel = 256; *nby = 210; return 0; case 39: *nel = 32; *nby = 17; return 0; }
  return -1;
}
static void deq_block(int t, const uint8_t* b, float* y) {
  switch (t) { case 2: deq_q4_0(b, y); break; case 8: deq_q8_0(b, y); break; case 14: deq_q6_k(b, y); break; case 39: deq_mxfp4(b, y); break;
               case 12: deq_q4_k(b, y); break; case 13: deq_q5_k(b, y); break;
               case 23: deq_iq4_xs(b, y); break; case 41: deq_q1_0(b, y); break;
               case 18: deq_iq3_xxs(b, y); break; case 21: deq_iq3_s(b, y); break; case 22: deq_iq2_s(b, y); break;
               case 3: deq_q4_1(b, y); break; case 6: deq_q5(b, y, 0); break; case 7: deq_q5(b, y, 1); break; }
}

/* ggml_data_to_tensor (tinygrad/llm/gguf.py:23): n_blocks blocks -> float32 */
int orc_dequant(int ggml_type, const uint8_t* blocks, int64_t n_blocks, float* out, int threads) {
  int nel, nby; if (type_geom(ggml_type, &nel, &nby)) return -1;
  (void)threads;
  #pragma omp parallel for num_threads(threads > 0 ? threads : 1) schedule(static)
  for (int64_t i = 0; i < n_blocks; i++) deq_block(ggml_type, blocks + i * nby, out + i * nel);
  return 0;
}

/* y[m,n] = sum_k x[m,k] * W[n,k], float32 accumulate in k order.
 * w_round_f16 = 1 applies the model path's fp16 cast of the dequantized weight (tinygrad/llm/model.py:376).
 * x_f16 = 1: x holds fp16 bits (config-1 style standalone matmul); products are then formed in float32 from the exact
 *            fp16 values (prod_round_f16 = 1 additionally rounds each product to fp16 as an fp16*fp16 Tensor multiply does,
 *            tinygrad/mixin/op.py:392). */
int orc_linear(int ggml_type, const uint8_t* w, const void* x, float* y, int M, int64_t N, int64_t K,
               int x_f16, int w_round_f16, int prod_round_f16, int threads) {
  int nel, nby; if (type_geom(ggml_type, &nel, &nby)) return -1;
  if (K % nel) return -2;
  const int64_t bpr = K / nel;
  float* xf = (float*)malloc(sizeof(float) * (size_t)M * K);
  for (int64_t i = 0; i < (int64_t)M * K; i++) xf[i] = x_f16 ? h2f(((const uint16_t*)x)[i]) : ((const float*)x)[i];
  #pragma omp parallel for num_threads(threads > 0 ? threads : 1) schedule(static)
  for (int64_t n = 0; n < N; n++) {
    float acc[8] = {0}; float wb[256];
    const uint8_t* row = w + n * bpr * nby;
    for (int64_t b = 0; b < bpr; b++) {
      deq_block(ggml_type, row + b * nby, wb);
      if (w_round_f16) round_f16_block(wb, nel);
      for (int m = 0; m < M; m++) {
        const float* xr = xf + (int64_t)m * K + b * nel; float a = acc[m];
        if (prod_round_f16) for (int j = 0; j < nel; j++) a += h2f(f2h(xr[j] * wb[j]));
        else for (int j = 0; j < nel; j++) a += xr[j] * wb[j];
        acc[m] = a;
      }
    }
    for (int m = 0; m < M; m++) y[(int64_t)m * N + n] = acc[m];
  }
  free(xf);
  return 0;
}

int orc_max_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}
