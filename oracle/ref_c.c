/* C restatement of the arithmetic of the three ref-eager kernels, independent of torch.
 * TEST INFRASTRUCTURE ONLY: loaded through ctypes by tests/ to cross-check oracle/oracle.py;
 * never linked into or called by the product library.
 *
 *   orc_e4m3_decode / orc_e4m3_encode : OCP float8 e4m3fn <-> float, RNE, |x|>464 -> NaN code
 *   orc_fp8_gemm_f64                  : examples/fp8_gemm.py:42-57 with a float64 accumulator
 *   orc_fp8_attention_f64             : examples/fp8_attention.py:54-105 for one (batch*head),
 *                                       single tile, float64 sums, fp32 score/exp2 path
 *   orc_moe_f64                       : examples/moe_matmul_ogs.py:125-148 (bf16 or fp16 bits in)
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

float orc_e4m3_decode(uint8_t c) {
  int s = c >> 7, e = (c >> 3) & 15, m = c & 7;
  float v;
  if (e == 15 && m == 7) return NAN;
  v = (e == 0) ? ldexpf((float)m, -9) : ldexpf((float)(8 + m), e - 10);
  return s ? -v : v;
}

uint8_t orc_e4m3_encode(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  uint8_t sign = (uint8_t)((u >> 24) & 0x80);
  float a = fabsf(f);
  if (isnan(f) || a > 464.0f) return sign | 0x7f;
  if (a >= 448.0f) return sign | 0x7e;
  /* quantum: 2^-9 below 2^-6, else 2^(floor(log2 a) - 3) */
  int ex;
  frexpf(a, &ex);           /* a = m * 2^ex, m in [0.5,1) -> floor(log2 a) = ex-1 */
  int q = (a < 0.015625f) ? -9 : (ex - 1 - 3);
  float scaled = ldexpf(a, -q);              /* exact */
  float r = nearbyintf(scaled);              /* default rounding mode: ties to even */
  float v = ldexpf(r, q);
  /* v is representable; find its code */
  if (v == 0.0f) return sign;
  int e2;
  float mant = frexpf(v, &e2);               /* v = mant * 2^e2, mant in [0.5,1) */
  int E = e2 - 1 + 7;
  if (E <= 0) return sign | (uint8_t)lrintf(ldexpf(v, 9));
  int M = (int)lrintf((mant * 2.0f - 1.0f) * 8.0f);
  return sign | (uint8_t)((E << 3) | M);
}

/* x: [M,K] codes row-major; y given as yt: [N,K] codes (i.e. y[k][n] = yt[n][k]); out fp64 */
void orc_fp8_gemm_f64(const uint8_t* x, const uint8_t* yt, double* out, int M, int N, int K) {
  for (int i = 0; i < M; ++i)
    for (int j = 0; j < N; ++j) {
      double acc = 0.0;
      for (int k = 0; k < K; ++k) acc += (double)orc_e4m3_decode(x[(size_t)i * K + k]) * (double)orc_e4m3_decode(yt[(size_t)j * K + k]);
      out[(size_t)i * N + j] = acc;
    }
}

/* one head: q,k [S,D] codes; vt [D,S] codes; out [S,D] float (before the final cast) */
void orc_fp8_attention_f64(const uint8_t* q, const uint8_t* k, const uint8_t* vt, float* out, int S, int D) {
  const float c = (float)((1.0 / sqrt((double)D)) * 1.44269504);
  float* s = (float*)malloc(sizeof(float) * S);
  for (int i = 0; i < S; ++i) {
    float m = -INFINITY;
    for (int j = 0; j < S; ++j) {
      double acc = 0.0;
      for (int d = 0; d < D; ++d) acc += (double)orc_e4m3_decode(q[(size_t)i * D + d]) * (double)orc_e4m3_decode(k[(size_t)j * D + d]);
      s[j] = (float)acc * c;            /* fp32 product with the fp32 scale */
      if (s[j] > m) m = s[j];
    }
    double l = 0.0;
    for (int j = 0; j < S; ++j) { s[j] = exp2f(s[j] - m); l += (double)s[j]; }
    for (int d = 0; d < D; ++d) {
      double acc = 0.0;
      for (int j = 0; j < S; ++j) acc += (double)orc_e4m3_decode(orc_e4m3_encode(s[j])) * (double)orc_e4m3_decode(vt[(size_t)d * S + j]);
      out[(size_t)i * D + d] = (float)(acc / l);
    }
  }
  free(s);
}

static float half_bits_to_float(uint16_t h, int is_bf16) {
  if (is_bf16) { uint32_t u = (uint32_t)h << 16; float f; memcpy(&f, &u, 4); return f; }
  int s = h >> 15, e = (h >> 10) & 31, m = h & 1023;
  float v;
  if (e == 0) v = ldexpf((float)m, -24);
  else if (e == 31) v = m ? NAN : INFINITY;
  else v = ldexpf((float)(1024 + m), e - 25);
  return s ? -v : v;
}

/* A [T,K], W [E,K,N] as 16-bit codes; expert[T]; out fp64 [T,N] (rows with expert<0 stay 0) */
void orc_moe_f64(const uint16_t* A, const uint16_t* W, const int32_t* expert, double* out, int T, int K, int N, int is_bf16) {
  for (int t = 0; t < T; ++t) {
    int e = expert[t];
    for (int n = 0; n < N; ++n) {
      double acc = 0.0;
      if (e >= 0)
        for (int k = 0; k < K; ++k)
          acc += (double)half_bits_to_float(A[(size_t)t * K + k], is_bf16) * (double)half_bits_to_float(W[((size_t)e * K + k) * N + n], is_bf16);
      out[(size_t)t * N + n] = acc;
    }
  }
}
