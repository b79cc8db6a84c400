/*
 * rwkv_oracle.c -- CPU restatement of the RWKV forward pass (see rwkv_oracle.h).
 *
 * TEST INFRASTRUCTURE ONLY: never linked into, or called from, the shipped library.
 *
 * Build: see oracle/Makefile (gcc -O2 -ffp-contract=off; F16C only accelerates the
 * half<->float conversions, whose results are identical to the portable code).
 */
#include "rwkv_oracle.h"

#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#ifdef __F16C__
#include <immintrin.h>
#endif

/* ======================================================================== */
/* binary16 arithmetic                                                       */
/* ======================================================================== */

orc_half orc_d2h(double d) {
  uint64_t b;
  memcpy(&b, &d, 8);
  uint16_t sign = (uint16_t)((b >> 48) & 0x8000u);
  int bexp = (int)((b >> 52) & 0x7FF);
  uint64_t man = b & 0xFFFFFFFFFFFFFull;
  if (bexp == 0x7FF) return (orc_half)(sign | 0x7C00u | (man ? 0x200u : 0u));
  if (bexp == 0) return sign; /* below 2^-1022: far under half's range */
  int e = bexp - 1023;
  if (e > 15) return (orc_half)(sign | 0x7C00u);
  man |= 1ull << 52; /* value = man * 2^(e-52) */
  int shift = (e >= -14) ? 42 : 42 + (-14 - e);
  if (shift >= 54) return sign;
  uint64_t q = man >> shift;
  uint64_t rem = man & ((1ull << shift) - 1);
  uint64_t half = 1ull << (shift - 1);
  if (rem > half || (rem == half && (q & 1))) q++;
  if (e >= -14) return (orc_half)(sign | (uint16_t)((((uint64_t)(e + 14)) << 10) + q));
  return (orc_half)(sign | (uint16_t)q);
}

orc_half orc_f2h(float f) { return orc_d2h((double)f); }

float orc_h2f(orc_half h) {
  uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1F;
  uint32_t man = h & 0x3FF;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else { /* subnormal: normalise */
      int sh = 0;
      while (!(man & 0x400)) {
        man <<= 1;
        sh++;
      }
      man &= 0x3FF;
      bits = sign | ((uint32_t)(127 - 15 - sh + 1) << 23) | (man << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7F800000u | (man << 13);
  } else {
    bits = sign | ((exp + 112) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

/* sums, differences and products of two halves are exact in double */
orc_half orc_hadd(orc_half a, orc_half b) { return orc_d2h((double)orc_h2f(a) + (double)orc_h2f(b)); }
orc_half orc_hsub(orc_half a, orc_half b) { return orc_d2h((double)orc_h2f(a) - (double)orc_h2f(b)); }
orc_half orc_hmul(orc_half a, orc_half b) { return orc_d2h((double)orc_h2f(a) * (double)orc_h2f(b)); }
/* a 53-bit quotient rounded again to 11 bits equals the directly rounded quotient
 * (double rounding is innocuous for division when p >= 2q+2). */
orc_half orc_hdiv(orc_half a, orc_half b) { return orc_d2h((double)orc_h2f(a) / (double)orc_h2f(b)); }

orc_half orc_hfma(orc_half a, orc_half b, orc_half c) {
  double p = (double)orc_h2f(a) * (double)orc_h2f(b); /* exact: 22 significant bits */
  double cc = (double)orc_h2f(c);
  double s = p + cc;
  if (isfinite(s)) {
    /* The sum may need more than 53 bits.  Recover the rounding error (TwoSum) and
     * turn the nearest-rounded sum into the round-to-odd one, so that the final
     * rounding to 11 bits is a correct single rounding. */
    double bb = s - p;
    double err = (p - (s - bb)) + (cc - bb);
    if (err != 0.0) {
      uint64_t bits;
      memcpy(&bits, &s, 8);
      if ((bits & 1) == 0) s = nextafter(s, err > 0 ? INFINITY : -INFINITY);
    }
  }
  return orc_d2h(s);
}

void orc_f2h_n(const float *src, orc_half *dst, size_t n) {
  size_t i = 0;
#ifdef __F16C__
  for (; i + 8 <= n; i += 8) {
    __m256 v = _mm256_loadu_ps(src + i);
    _mm_storeu_si128((__m128i *)(dst + i), _mm256_cvtps_ph(v, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC));
  }
#endif
  for (; i < n; i++) dst[i] = orc_f2h(src[i]);
}

void orc_h2f_n(const orc_half *src, float *dst, size_t n) {
  size_t i = 0;
#ifdef __F16C__
  for (; i + 8 <= n; i += 8) {
    __m128i v = _mm_loadu_si128((const __m128i *)(src + i));
    _mm256_storeu_ps(dst + i, _mm256_cvtph_ps(v));
  }
#endif
  for (; i < n; i++) dst[i] = orc_h2f(src[i]);
}

static void *xmalloc(size_t n) {
  void *p = malloc(n ? n : 1);
  if (!p) abort();
  return p;
}

/* ======================================================================== */
/* primitive ops                                                             */
/* ======================================================================== */

static void row_stats(const float *x, int cols, float *mean_out, float *inv_out) {
  double sum = 0.0;
  for (int i = 0; i < cols; i++) sum += x[i];
  double mean = sum / cols;
  double m2 = 0.0;
  for (int i = 0; i < cols; i++) {
    double d = x[i] - mean;
    m2 += d * d;
  }
  float var = (float)(m2 / cols);
  if (var < 0.f) var = 0.f;
  *mean_out = (float)mean;
  *inv_out = 1.0f / sqrtf(var + 1e-5f);
}

void orc_layernorm_f16(const orc_half *x, const orc_half *gamma, const orc_half *beta,
                       orc_half *y, int rows, int cols) {
  float *xf = (float *)xmalloc(sizeof(float) * (size_t)cols);
  for (int r = 0; r < rows; r++) {
    orc_h2f_n(x + (size_t)r * cols, xf, (size_t)cols);
    float mean, inv;
    row_stats(xf, cols, &mean, &inv);
    for (int i = 0; i < cols; i++) {
      orc_half nh = orc_f2h((xf[i] - mean) * inv);
      y[(size_t)r * cols + i] = orc_hadd(orc_hmul(nh, gamma[i]), beta[i]);
    }
  }
  free(xf);
}

void orc_layernorm_f32(const float *x, const float *gamma, const float *beta, float *y,
                       int rows, int cols) {
  for (int r = 0; r < rows; r++) {
    const float *xr = x + (size_t)r * cols;
    float mean, inv;
    row_stats(xr, cols, &mean, &inv);
    for (int i = 0; i < cols; i++) y[(size_t)r * cols + i] = (xr[i] - mean) * inv * gamma[i] + beta[i];
  }
}

void orc_groupnorm_f32(const float *x, int groups, const float *gamma, const float *beta,
                       float *y, int rows, int cols) {
  int gs = cols / groups;
  for (int r = 0; r < rows; r++) {
    for (int g = 0; g < groups; g++) {
      const float *xr = x + (size_t)r * cols + (size_t)g * gs;
      float *yr = y + (size_t)r * cols + (size_t)g * gs;
      float mean, inv;
      row_stats(xr, gs, &mean, &inv);
      for (int i = 0; i < gs; i++) yr[i] = (xr[i] - mean) * inv * gamma[g * gs + i] + beta[g * gs + i];
    }
  }
}

void orc_mix_f16(const orc_half *xx, const orc_half *sx, const orc_half *mix, orc_half *out,
                 int rows, int cols) {
  const orc_half one = 0x3C00;
  for (int r = 0; r < rows; r++)
    for (int i = 0; i < cols; i++) {
      size_t idx = (size_t)r * cols + i;
      orc_half m = mix[i];
      out[idx] = orc_hadd(orc_hmul(xx[idx], m), orc_hmul(sx[idx], orc_hsub(one, m)));
    }
}

void orc_mix_f32(const float *xx, const float *sx, const float *mix, float *out, int rows,
                 int cols) {
  for (int r = 0; r < rows; r++)
    for (int i = 0; i < cols; i++) {
      size_t idx = (size_t)r * cols + i;
      out[idx] = xx[idx] * mix[i] + sx[idx] * (1.0f - mix[i]);
    }
}

/* ------------------------------------------------------------------------
 * uint8 weights in the one-token products.  The ChatRWKV scheme this format comes from has two
 * evaluations of the same dequantisation formula: its matrix x matrix path expands the codes to a
 * binary16 matrix first (orc_dequant_u8: one rounding of w^ to half), its vector x matrix kernel
 * forms every weight in fp32 and multiplies it unrounded (rwkv pip package 0.8.x,
 * rwkv/cuda/operators.cu, kernel_mm_one_fp16i8 -- not part of the reference tree, restated from its
 * published source: PARITY UNPINNED by the reference).  orc_gemv_u8 is the second one:
 *   y[n] = sum_k x[k] * fmaf(q[k][n], (rx[n]/255)*ry[k], mx[n]+my[k])      (each weight in fp32,
 * products and sum exact in double, one rounding of the sum to fp32).
 * A binary16 matrix handed to orc_gemm_f16 with T == 1 is multiplied this way when its codes have
 * been registered with orc_register_u8 (keyed by the matrix pointer); with T > 1 the binary16
 * matrix itself is used.
 * ------------------------------------------------------------------------ */
static int g_acc_mode = ORC_ACC_EXACT;
void orc_set_accumulation(int mode) { g_acc_mode = mode; }

typedef struct {
  const orc_half *W;
  const uint8_t *q;
  const orc_half *mx, *rx, *my, *ry;
} orc_u8_rec;
static orc_u8_rec *g_u8 = NULL;
static size_t g_u8_n = 0, g_u8_cap = 0;

void orc_register_u8(const orc_half *W, const uint8_t *q, const orc_half *mx, const orc_half *rx,
                     const orc_half *my, const orc_half *ry) {
  for (size_t i = 0; i < g_u8_n; i++)
    if (g_u8[i].W == W) {
      g_u8[i] = (orc_u8_rec){W, q, mx, rx, my, ry};
      return;
    }
  if (g_u8_n == g_u8_cap) {
    g_u8_cap = g_u8_cap ? 2 * g_u8_cap : 64;
    g_u8 = (orc_u8_rec *)realloc(g_u8, g_u8_cap * sizeof(orc_u8_rec));
    if (!g_u8) abort();
  }
  g_u8[g_u8_n++] = (orc_u8_rec){W, q, mx, rx, my, ry};
}

void orc_unregister_u8(const orc_half *W) {
  for (size_t i = 0; i < g_u8_n; i++)
    if (g_u8[i].W == W) {
      g_u8[i] = g_u8[--g_u8_n];
      return;
    }
}

void orc_gemv_u8(const orc_half *x, const uint8_t *q, const orc_half *mx, const orc_half *rx,
                 const orc_half *my, const orc_half *ry, float *y, int K, int N) {
  float *xf = (float *)xmalloc(sizeof(float) * (size_t)K);
  float *ryf = (float *)xmalloc(sizeof(float) * (size_t)K);
  float *myf = (float *)xmalloc(sizeof(float) * (size_t)K);
  orc_h2f_n(x, xf, (size_t)K);
  orc_h2f_n(ry, ryf, (size_t)K);
  orc_h2f_n(my, myf, (size_t)K);
  int nblocks = (N + 63) / 64;
#pragma omp parallel for schedule(static)
  for (int nb = 0; nb < nblocks; nb++) {
    int n0 = nb * 64, n1 = n0 + 64 < N ? n0 + 64 : N;
    double acc[64];
    float facc[64];
    float c[64], m[64];
    for (int j = 0; j < n1 - n0; j++) {
      acc[j] = 0.0;
      facc[j] = 0.f;
      c[j] = orc_h2f(rx[n0 + j]) / 255.0f;
      m[j] = orc_h2f(mx[n0 + j]);
    }
    /* the same weights either way; only the accumulation differs (one loop per mode: the mode is fixed for a call) */
    if (g_acc_mode == ORC_ACC_F32_SEQUENTIAL) {
      for (int k = 0; k < K; k++) {
        const uint8_t *qr = q + (size_t)k * N + n0;
        for (int j = 0; j < n1 - n0; j++) {
          const float a = c[j] * ryf[k];
          const float b = m[j] + myf[k];
          const float w32 = fmaf((float)qr[j], a, b);
          facc[j] += xf[k] * w32; /* fp32 products and sums, ascending k */
        }
      }
    } else {
      for (int k = 0; k < K; k++) {
        const uint8_t *qr = q + (size_t)k * N + n0;
        const double xk = (double)xf[k];
        for (int j = 0; j < n1 - n0; j++) {
          const float a = c[j] * ryf[k];
          const float b = m[j] + myf[k];
          const float w32 = fmaf((float)qr[j], a, b);
          acc[j] += xk * (double)w32;
        }
      }
    }
    for (int j = 0; j < n1 - n0; j++)
      y[n0 + j] = g_acc_mode == ORC_ACC_F32_SEQUENTIAL ? facc[j] : (float)acc[j];
  }
  free(xf); free(ryf); free(myf);
}

#define NB 256 /* column block */
#define TB 8   /* row block    */

void orc_gemm_f16(const orc_half *x, const orc_half *W, float *y_f32, orc_half *y_f16, int T,
                  int K, int N) {
  if (T == 1) /* registered uint8 codes: the one-token product multiplies the unrounded fp32 weight */
    for (size_t i = 0; i < g_u8_n; i++)
      if (g_u8[i].W == W) {
        float *y = y_f32 ? y_f32 : (float *)xmalloc(sizeof(float) * (size_t)N);
        orc_gemv_u8(x, g_u8[i].q, g_u8[i].mx, g_u8[i].rx, g_u8[i].my, g_u8[i].ry, y, K, N);
        if (y_f16) orc_f2h_n(y, y_f16, (size_t)N);
        if (!y_f32) free(y);
        return;
      }
  float *xf = (float *)xmalloc(sizeof(float) * (size_t)T * K);
  orc_h2f_n(x, xf, (size_t)T * K);
  int nblocks = (N + NB - 1) / NB;
#pragma omp parallel for schedule(static)
  for (int nb = 0; nb < nblocks; nb++) {
    int n0 = nb * NB, n1 = n0 + NB < N ? n0 + NB : N, w = n1 - n0;
    /* The reference accumulates in fp32 in an order that is cuBLAS's own (matmul.cpp:38-42): every
     * such order lies within its own rounding error of the exact sum.  The oracle returns the centre
     * of that family -- the exact sum (products of two halves and their sum are exact in double for
     * any K here) rounded once to fp32 -- so that a comparison measures the other side's error only. */
    double acc[TB][NB];
    float wrow[NB], out[NB];
    if (g_acc_mode == ORC_ACC_F32_SEQUENTIAL) { /* another member of the family: fp32, ascending k */
      float facc[TB][NB];
      for (int t0 = 0; t0 < T; t0 += TB) {
        int tn = t0 + TB < T ? TB : T - t0;
        for (int t = 0; t < tn; t++)
          for (int j = 0; j < w; j++) facc[t][j] = 0.f;
        for (int k = 0; k < K; k++) {
          orc_h2f_n(W + (size_t)k * N + n0, wrow, (size_t)w);
          for (int t = 0; t < tn; t++) {
            float xk = xf[(size_t)(t0 + t) * K + k];
            for (int j = 0; j < w; j++) facc[t][j] += xk * wrow[j]; /* product exact in fp32 */
          }
        }
        for (int t = 0; t < tn; t++) {
          if (y_f32) memcpy(y_f32 + (size_t)(t0 + t) * N + n0, facc[t], sizeof(float) * (size_t)w);
          if (y_f16) orc_f2h_n(facc[t], y_f16 + (size_t)(t0 + t) * N + n0, (size_t)w);
        }
      }
      continue;
    }
    for (int t0 = 0; t0 < T; t0 += TB) {
      int tn = t0 + TB < T ? TB : T - t0;
      for (int t = 0; t < tn; t++)
        for (int j = 0; j < w; j++) acc[t][j] = 0.0;
      for (int k = 0; k < K; k++) {
        orc_h2f_n(W + (size_t)k * N + n0, wrow, (size_t)w);
        for (int t = 0; t < tn; t++) {
          double xk = (double)xf[(size_t)(t0 + t) * K + k];
          for (int j = 0; j < w; j++) acc[t][j] += xk * (double)wrow[j];
        }
      }
      for (int t = 0; t < tn; t++) {
        for (int j = 0; j < w; j++) out[j] = (float)acc[t][j];
        if (y_f32) memcpy(y_f32 + (size_t)(t0 + t) * N + n0, out, sizeof(float) * (size_t)w);
        if (y_f16) orc_f2h_n(out, y_f16 + (size_t)(t0 + t) * N + n0, (size_t)w);
      }
    }
  }
  free(xf);
}

void orc_gemm_f32(const float *x, const float *W, float *y, int T, int K, int N) {
  int nblocks = (N + NB - 1) / NB;
#pragma omp parallel for schedule(static)
  for (int nb = 0; nb < nblocks; nb++) {
    int n0 = nb * NB, n1 = n0 + NB < N ? n0 + NB : N, w = n1 - n0;
    float acc[TB][NB];
    for (int t0 = 0; t0 < T; t0 += TB) {
      int tn = t0 + TB < T ? TB : T - t0;
      for (int t = 0; t < tn; t++)
        for (int j = 0; j < w; j++) acc[t][j] = 0.f;
      for (int k = 0; k < K; k++) {
        const float *wrow = W + (size_t)k * N + n0;
        for (int t = 0; t < tn; t++) {
          float xk = x[(size_t)(t0 + t) * K + k];
          for (int j = 0; j < w; j++) acc[t][j] += xk * wrow[j];
        }
      }
      for (int t = 0; t < tn; t++) memcpy(y + (size_t)(t0 + t) * N + n0, acc[t], sizeof(float) * (size_t)w);
    }
  }
}

void orc_sigmoid_f16(orc_half *x, size_t n) {
  for (size_t i = 0; i < n; i++) {
    /* the reference evaluates in double, narrows to float, then to half */
    double s = 1.0 / (1.0 + exp(-(double)orc_h2f(x[i])));
    x[i] = orc_f2h((float)s);
  }
}

void orc_relu_square_f16(orc_half *x, size_t n) {
  for (size_t i = 0; i < n; i++) {
    float f = orc_h2f(x[i]);
    x[i] = (f > 0.f) ? orc_hmul(x[i], x[i]) : (orc_half)0;
  }
}

void orc_silu_f16(orc_half *x, size_t n) {
  const orc_half one = 0x3C00;
  for (size_t i = 0; i < n; i++) {
    orc_half e = orc_f2h(expf(-orc_h2f(x[i])));
    x[i] = orc_hdiv(x[i], orc_hadd(one, e));
  }
}

void orc_wkv4_one_f16(const float *t_first, const float *t_decay, const float *k,
                      const float *v, float *aa, float *bb, float *pp, orc_half *r, int n) {
  for (int i = 0; i < n; i++) {
    float ww = t_first[i] + k[i];
    float pp_ = pp[i];
    float p_ = (pp_ > ww) ? pp_ : ww;
    float e1 = expf(pp_ - p_);
    float e2 = expf(ww - p_);
    float aa_ = aa[i], bb_ = bb[i], v_ = v[i];
    float wkv = (e1 * aa_ + e2 * v_) / (e1 * bb_ + e2);
    r[i] = orc_hmul(r[i], orc_f2h(wkv));
    ww = t_decay[i] + pp_;
    float k_ = k[i];
    p_ = (ww > k_) ? ww : k_;
    e1 = expf(ww - p_);
    e2 = expf(k_ - p_);
    aa[i] = e1 * aa_ + e2 * v_;
    bb[i] = e1 * bb_ + e2;
    pp[i] = p_;
  }
}

/* fp32 form of the same step, following kernels/default/att.cpp:31-44 */
static void wkv4_one_f32(const float *t_first, const float *t_decay, const float *k,
                         const float *v, float *aa, float *bb, float *pp, float *r, int n) {
  for (int i = 0; i < n; i++) {
    float ww = t_first[i] + k[i];
    float pp_ = pp[i];
    float p_ = fmaxf(pp_, ww);
    float e1 = expf(pp_ - p_), e2 = expf(ww - p_);
    float aa_ = aa[i], bb_ = bb[i], v_ = v[i];
    float wkv = (e1 * aa_ + e2 * v_) / (e1 * bb_ + e2);
    r[i] = r[i] * wkv;
    ww = t_decay[i] + pp_;
    p_ = fmaxf(ww, k[i]);
    e1 = expf(ww - p_);
    e2 = expf(k[i] - p_);
    aa[i] = e1 * aa_ + e2 * v_;
    bb[i] = e1 * bb_ + e2;
    pp[i] = p_;
  }
}

/* ======================================================================== */
/* uint8 dequantisation                                                      */
/* ======================================================================== */

orc_half orc_dequant_u8_scalar(uint8_t q, orc_half mx, orc_half rx, orc_half my, orc_half ry) {
  float c = orc_h2f(rx) / 255.0f;
  float a = c * orc_h2f(ry);
  float b = orc_h2f(mx) + orc_h2f(my);
  return orc_f2h(fmaf((float)q, a, b));
}

void orc_dequant_u8(const uint8_t *q, const orc_half *mx, const orc_half *rx,
                    const orc_half *my, const orc_half *ry, orc_half *W, int K, int N) {
#pragma omp parallel for schedule(static)
  for (int k = 0; k < K; k++)
    for (int n = 0; n < N; n++)
      W[(size_t)k * N + n] = orc_dequant_u8_scalar(q[(size_t)k * N + n], mx[n], rx[n], my[k], ry[k]);
}

/* ======================================================================== */
/* layer-level ops, fp16 emulation                                           */
/* ======================================================================== */

static void shift_rows_f16(const orc_half *sx, const orc_half *xx, orc_half *out, int T, int C) {
  /* token shift: row 0 = state, row t = xx[t-1]  (ffn_seq.cu:71-72, att_seq.cu:380-381) */
  memcpy(out, sx, sizeof(orc_half) * (size_t)C);
  if (T > 1) memcpy(out + C, xx, sizeof(orc_half) * (size_t)(T - 1) * C);
}

void orc_att_seq_v4_f16(const orc_half *x, const orc_half *sx, float *aa, float *bb, float *pp,
                        const orc_half *ln_w, const orc_half *ln_b, const orc_half *k_mix,
                        const orc_half *v_mix, const orc_half *r_mix, const float *t_decay,
                        const float *t_first, const orc_half *kw, const orc_half *vw,
                        const orc_half *rw, const orc_half *ow, orc_half *x_out,
                        orc_half *xx_last_out, int T, int C) {
  size_t n = (size_t)T * C;
  orc_half *xx = (orc_half *)xmalloc(2 * n), *sh = (orc_half *)xmalloc(2 * n);
  orc_half *kx = (orc_half *)xmalloc(2 * n), *vx = (orc_half *)xmalloc(2 * n), *rx = (orc_half *)xmalloc(2 * n);
  float *k = (float *)xmalloc(4 * n), *v = (float *)xmalloc(4 * n);
  orc_half *r = (orc_half *)xmalloc(2 * n), *out = (orc_half *)xmalloc(2 * n);
  orc_layernorm_f16(x, ln_w, ln_b, xx, T, C);
  shift_rows_f16(sx, xx, sh, T, C);
  orc_mix_f16(xx, sh, k_mix, kx, T, C);
  orc_mix_f16(xx, sh, v_mix, vx, T, C);
  orc_mix_f16(xx, sh, r_mix, rx, T, C);
  orc_gemm_f16(kx, kw, k, NULL, T, C, C);
  orc_gemm_f16(vx, vw, v, NULL, T, C, C);
  orc_gemm_f16(rx, rw, NULL, r, T, C, C);
  orc_sigmoid_f16(r, n);
  for (int t = 0; t < T; t++)
    orc_wkv4_one_f16(t_first, t_decay, k + (size_t)t * C, v + (size_t)t * C, aa, bb, pp,
                     r + (size_t)t * C, C);
  orc_gemm_f16(r, ow, NULL, out, T, C, C);
  for (size_t i = 0; i < n; i++) x_out[i] = orc_hadd(x[i], out[i]);
  memcpy(xx_last_out, xx + (size_t)(T - 1) * C, sizeof(orc_half) * (size_t)C);
  free(xx); free(sh); free(kx); free(vx); free(rx); free(k); free(v); free(r); free(out);
}

void orc_att_one_v4_f16(const orc_half *x, const orc_half *sx, float *aa, float *bb, float *pp,
                        const orc_half *ln_w, const orc_half *ln_b, const orc_half *k_mix,
                        const orc_half *v_mix, const orc_half *r_mix, const float *t_decay,
                        const float *t_first, const orc_half *kw, const orc_half *vw,
                        const orc_half *rw, const orc_half *ow, orc_half *x_out,
                        orc_half *xx_out, int C) {
  orc_att_seq_v4_f16(x, sx, aa, bb, pp, ln_w, ln_b, k_mix, v_mix, r_mix, t_decay, t_first, kw,
                     vw, rw, ow, x_out, xx_out, 1, C);
}

void orc_ffn_seq_f16(const orc_half *x, const orc_half *sx, const orc_half *ln_w,
                     const orc_half *ln_b, const orc_half *k_mix, const orc_half *r_mix,
                     const orc_half *kw, const orc_half *vw, const orc_half *rw, orc_half *x_out,
                     orc_half *xx_last_out, int T, int C, int F) {
  size_t n = (size_t)T * C, nf = (size_t)T * F;
  orc_half *xx = (orc_half *)xmalloc(2 * n), *sh = (orc_half *)xmalloc(2 * n);
  orc_half *kx = (orc_half *)xmalloc(2 * n), *rx = (orc_half *)xmalloc(2 * n);
  orc_half *r = (orc_half *)xmalloc(2 * n), *vx = (orc_half *)xmalloc(2 * nf), *out = (orc_half *)xmalloc(2 * n);
  orc_layernorm_f16(x, ln_w, ln_b, xx, T, C);
  shift_rows_f16(sx, xx, sh, T, C);
  orc_mix_f16(xx, sh, k_mix, kx, T, C);
  orc_mix_f16(xx, sh, r_mix, rx, T, C);
  orc_gemm_f16(rx, rw, NULL, r, T, C, C);
  orc_sigmoid_f16(r, n);
  orc_gemm_f16(kx, kw, NULL, vx, T, C, F);
  orc_relu_square_f16(vx, nf);
  orc_gemm_f16(vx, vw, NULL, out, T, F, C);
  for (size_t i = 0; i < n; i++) x_out[i] = orc_hfma(out[i], r[i], x[i]);
  memcpy(xx_last_out, xx + (size_t)(T - 1) * C, sizeof(orc_half) * (size_t)C);
  free(xx); free(sh); free(kx); free(rx); free(r); free(vx); free(out);
}

void orc_ffn_one_f16(const orc_half *x, const orc_half *sx, const orc_half *ln_w,
                     const orc_half *ln_b, const orc_half *k_mix, const orc_half *r_mix,
                     const orc_half *kw, const orc_half *vw, const orc_half *rw, orc_half *x_out,
                     orc_half *xx_out, int C, int F) {
  orc_ffn_seq_f16(x, sx, ln_w, ln_b, k_mix, r_mix, kw, vw, rw, x_out, xx_out, 1, C, F);
}

/* One token of the RWKV-5.1/5.2 state update on state s[h][i(key)][j(value)]:
 *   a_ij = k_i v_j ; tmp = u_i a_ij + s_ij ; out_j = sum_i r_i tmp_ij ; s_ij = w_i s_ij + a_ij
 * with products and sums rounded separately (kernels/cuda/att.cu:64-81, :296-311). */
static void wkv5_one_f32(float *s, const float *r, const float *k, const float *v, const float *w,
                         const float *u, float *out, int H, int S) {
  for (int h = 0; h < H; h++) {
    float *sh = s + (size_t)h * S * S;
    const float *rh = r + h * S, *kh = k + h * S, *vh = v + h * S, *wh = w + h * S, *uh = u + h * S;
    float *oh = out + h * S;
    for (int j = 0; j < S; j++) oh[j] = 0.f;
    for (int i = 0; i < S; i++) {
      for (int j = 0; j < S; j++) {
        float a = kh[i] * vh[j];
        float ua = uh[i] * a;
        float tmp = ua + sh[i * S + j];
        float ws = wh[i] * sh[i * S + j];
        sh[i * S + j] = ws + a;
        oh[j] += rh[i] * tmp;
      }
    }
  }
}

void orc_wkv5_2_seq_f32(float *s, const float *r, const float *k, const float *v,
                        const float *w, const float *u, float *y, int T, int H, int S) {
  /* att_seq.cu:284-318: thread i owns value index i and loops over key index j;
   * on the [key][value] state that is s[j][i]. */
  int C = H * S;
  for (int t = 0; t < T; t++) {
    for (int h = 0; h < H; h++) {
      float *sh = s + (size_t)h * S * S;
      const float *rt = r + (size_t)t * C + h * S, *kt = k + (size_t)t * C + h * S,
                  *vt = v + (size_t)t * C + h * S;
      const float *wh = w + h * S, *uh = u + h * S;
      for (int i = 0; i < S; i++) {
        float vi = vt[i], acc = 0.f;
        for (int j = 0; j < S; j++) {
          float x = kt[j] * vi;
          acc += rt[j] * (uh[j] * x + sh[j * S + i]);
          sh[j * S + i] = sh[j * S + i] * wh[j] + x;
        }
        y[(size_t)t * C + h * S + i] = acc;
      }
    }
  }
}

static void att_v5_2_tail_f16(const orc_half *x, const float *wkv_out, const float *lx_w,
                              const float *lx_b, const orc_half *g, const orc_half *ow,
                              orc_half *x_out, int T, int C, int H) {
  /* GroupNorm(fp32) -> half -> * g -> GEMM(ow) -> + x   (att.cu:314-329, att_seq.cu:406-416) */
  size_t n = (size_t)T * C;
  float *gn = (float *)xmalloc(4 * n);
  orc_half *gh = (orc_half *)xmalloc(2 * n), *out = (orc_half *)xmalloc(2 * n);
  orc_groupnorm_f32(wkv_out, H, lx_w, lx_b, gn, T, C);
  orc_f2h_n(gn, gh, n);
  if (g) /* RWKV-5.0 has no gate: att.cu:258-259 */
    for (size_t i = 0; i < n; i++) gh[i] = orc_hmul(gh[i], g[i]);
  orc_gemm_f16(gh, ow, NULL, out, T, C, C);
  for (size_t i = 0; i < n; i++) x_out[i] = orc_hadd(x[i], out[i]);
  free(gn); free(gh); free(out);
}

static void att_v5_2_f16(const orc_half *x, const orc_half *sx, float *s, const orc_half *ln_w,
                         const orc_half *ln_b, const float *lx_w, const float *lx_b,
                         const orc_half *k_mix, const orc_half *v_mix, const orc_half *r_mix,
                         const orc_half *g_mix, const float *t_decay, const float *t_first,
                         const orc_half *kw, const orc_half *vw, const orc_half *rw,
                         const orc_half *gw, const orc_half *ow, orc_half *x_out,
                         orc_half *xx_last_out, int T, int C, int H, int scan_form) {
  size_t n = (size_t)T * C;
  int S = C / H;
  orc_half *xx = (orc_half *)xmalloc(2 * n), *sh = (orc_half *)xmalloc(2 * n);
  orc_half *kx = (orc_half *)xmalloc(2 * n), *vx = (orc_half *)xmalloc(2 * n);
  orc_half *rx = (orc_half *)xmalloc(2 * n), *gx = (orc_half *)xmalloc(2 * n), *g = (orc_half *)xmalloc(2 * n);
  float *k = (float *)xmalloc(4 * n), *v = (float *)xmalloc(4 * n), *r = (float *)xmalloc(4 * n);
  float *y = (float *)xmalloc(4 * n);
  orc_layernorm_f16(x, ln_w, ln_b, xx, T, C);
  shift_rows_f16(sx, xx, sh, T, C);
  orc_mix_f16(xx, sh, k_mix, kx, T, C);
  orc_mix_f16(xx, sh, v_mix, vx, T, C);
  orc_mix_f16(xx, sh, r_mix, rx, T, C);
  orc_mix_f16(xx, sh, g_mix, gx, T, C);
  orc_gemm_f16(kx, kw, k, NULL, T, C, C);
  orc_gemm_f16(vx, vw, v, NULL, T, C, C);
  orc_gemm_f16(rx, rw, r, NULL, T, C, C);
  orc_gemm_f16(gx, gw, NULL, g, T, C, C);
  orc_silu_f16(g, n);
  if (scan_form) {
    orc_wkv5_2_seq_f32(s, r, k, v, t_decay, t_first, y, T, H, S);
  } else {
    for (int t = 0; t < T; t++)
      wkv5_one_f32(s, r + (size_t)t * C, k + (size_t)t * C, v + (size_t)t * C, t_decay, t_first,
                   y + (size_t)t * C, H, S);
  }
  att_v5_2_tail_f16(x, y, lx_w, lx_b, g, ow, x_out, T, C, H);
  memcpy(xx_last_out, xx + (size_t)(T - 1) * C, sizeof(orc_half) * (size_t)C);
  free(xx); free(sh); free(kx); free(vx); free(rx); free(gx); free(g); free(k); free(v); free(r); free(y);
}

void orc_att_one_v5_1_f16(const orc_half *x, const orc_half *sx, float *s, const orc_half *ln_w,
                          const orc_half *ln_b, const float *lx_w, const float *lx_b,
                          const orc_half *k_mix, const orc_half *v_mix, const orc_half *r_mix,
                          const orc_half *g_mix, const float *t_decay, const float *t_first,
                          const orc_half *kw, const orc_half *vw, const orc_half *rw,
                          const orc_half *gw, const orc_half *ow, orc_half *x_out,
                          orc_half *xx_out, int C, int H) {
  att_v5_2_f16(x, sx, s, ln_w, ln_b, lx_w, lx_b, k_mix, v_mix, r_mix, g_mix, t_decay, t_first, kw,
               vw, rw, gw, ow, x_out, xx_out, 1, C, H, 0);
}

void orc_att_seq_v5_2_f16(const orc_half *x, const orc_half *sx, float *s, const orc_half *ln_w,
                          const orc_half *ln_b, const float *lx_w, const float *lx_b,
                          const orc_half *k_mix, const orc_half *v_mix, const orc_half *r_mix,
                          const orc_half *g_mix, const float *t_decay, const float *t_first,
                          const orc_half *kw, const orc_half *vw, const orc_half *rw,
                          const orc_half *gw, const orc_half *ow, orc_half *x_out,
                          orc_half *xx_last_out, int T, int C, int H) {
  att_v5_2_f16(x, sx, s, ln_w, ln_b, lx_w, lx_b, k_mix, v_mix, r_mix, g_mix, t_decay, t_first, kw,
               vw, rw, gw, ow, x_out, xx_last_out, T, C, H, 1);
}

/* RWKV-5.0 sequence recurrence in the reference's matrix form (att_seq.cu:181-243), per head
 * with scalar decay w and bonus u:
 *   out_t = sum_{i<t} (r_t.k_i) w^(t-1-i) v_i + u (r_t.k_t) v_t + (r_t S) w^t
 *   S'    = w^T S + sum_i w^(T-1-i) k_i v_i^T
 * powers through powf as the reference's __powf functors (att_seq.cu:142-155). */
void orc_wkv5_seq_matrix_f32(float *s, const float *r, const float *k, const float *v,
                             const float *w, const float *u, float *y, int T, int H, int S) {
  int C = H * S;
  float *rk = (float *)xmalloc(4 * (size_t)T * T), *rs = (float *)xmalloc(4 * (size_t)T * S);
  float *sn = (float *)xmalloc(4 * (size_t)S * S);
  for (int h = 0; h < H; h++) {
    float *sh = s + (size_t)h * S * S;
    const float wh = w[h], uh = u[h];
    for (int t = 0; t < T; t++) {
      const float *rt = r + (size_t)t * C + h * S;
      for (int i = 0; i <= t; i++) {
        const float *ki = k + (size_t)i * C + h * S;
        float acc = 0.f;
        for (int c = 0; c < S; c++) acc += rt[c] * ki[c];
        float wt = i == t ? uh : powf(wh, (float)(t - 1 - i)); /* att_seq.cu:193-201 */
        rk[(size_t)t * T + i] = acc * wt;
      }
      for (int j = 0; j < S; j++) {
        float acc = 0.f;
        for (int c = 0; c < S; c++) acc += rt[c] * sh[c * S + j];
        rs[(size_t)t * S + j] = acc * powf(wh, (float)t); /* wb: att_seq.cu:192,222-225 */
      }
    }
    for (int t = 0; t < T; t++)
      for (int j = 0; j < S; j++) {
        float acc = 0.f;
        for (int i = 0; i <= t; i++) acc += rk[(size_t)t * T + i] * v[(size_t)i * C + h * S + j];
        y[(size_t)t * C + h * S + j] = acc + rs[(size_t)t * S + j]; /* att_seq.cu:227-231 */
      }
    const float wT = powf(wh, (float)T); /* att_seq.cu:183-186 */
    for (int c = 0; c < S; c++)
      for (int j = 0; j < S; j++) {
        float acc = 0.f;
        for (int i = 0; i < T; i++)
          acc += (k[(size_t)i * C + h * S + c] * powf(wh, (float)(T - 1 - i))) * v[(size_t)i * C + h * S + j];
        sn[c * S + j] = wT * sh[c * S + j] + acc; /* att_seq.cu:232-243 */
      }
    memcpy(sh, sn, 4 * (size_t)S * S);
  }
  free(rk); free(rs); free(sn);
}

/* RWKV-5.0 attention: one token kernels/cuda/att.cu:219-265,362-391 (matrix_form 0),
 * sequence kernels/cuda/att_seq.cu:158-256,425-462 (matrix_form 1).  t_decay, t_first [H]. */
static void att_v5_0_f16(const orc_half *x, const orc_half *sx, float *s, const orc_half *ln_w,
                         const orc_half *ln_b, const float *lx_w, const float *lx_b,
                         const orc_half *k_mix, const orc_half *v_mix, const orc_half *r_mix,
                         const float *t_decay, const float *t_first, const orc_half *kw,
                         const orc_half *vw, const orc_half *rw, const orc_half *ow,
                         orc_half *x_out, orc_half *xx_last_out, int T, int C, int H,
                         int matrix_form) {
  size_t n = (size_t)T * C;
  int S = C / H;
  orc_half *xx = (orc_half *)xmalloc(2 * n), *sh = (orc_half *)xmalloc(2 * n);
  orc_half *kx = (orc_half *)xmalloc(2 * n), *vx = (orc_half *)xmalloc(2 * n), *rx = (orc_half *)xmalloc(2 * n);
  float *k = (float *)xmalloc(4 * n), *v = (float *)xmalloc(4 * n), *r = (float *)xmalloc(4 * n);
  float *y = (float *)xmalloc(4 * n);
  orc_layernorm_f16(x, ln_w, ln_b, xx, T, C);
  shift_rows_f16(sx, xx, sh, T, C);
  orc_mix_f16(xx, sh, k_mix, kx, T, C);
  orc_mix_f16(xx, sh, v_mix, vx, T, C);
  orc_mix_f16(xx, sh, r_mix, rx, T, C);
  orc_gemm_f16(kx, kw, k, NULL, T, C, C);
  orc_gemm_f16(vx, vw, v, NULL, T, C, C);
  orc_gemm_f16(rx, rw, r, NULL, T, C, C);
  if (matrix_form) {
    orc_wkv5_seq_matrix_f32(s, r, k, v, t_decay, t_first, y, T, H, S);
  } else {
    /* OneV5MulAdd indexes t_first, t_decay by i / (S*S) (att.cu:70,73): one value per head */
    float *wx = (float *)xmalloc(4 * (size_t)C), *ux = (float *)xmalloc(4 * (size_t)C);
    for (int i = 0; i < C; i++) { wx[i] = t_decay[i / S]; ux[i] = t_first[i / S]; }
    for (int t = 0; t < T; t++)
      wkv5_one_f32(s, r + (size_t)t * C, k + (size_t)t * C, v + (size_t)t * C, wx, ux, y + (size_t)t * C, H, S);
    free(wx); free(ux);
  }
  att_v5_2_tail_f16(x, y, lx_w, lx_b, NULL, ow, x_out, T, C, H);
  memcpy(xx_last_out, xx + (size_t)(T - 1) * C, sizeof(orc_half) * (size_t)C);
  free(xx); free(sh); free(kx); free(vx); free(rx); free(k); free(v); free(r); free(y);
}

void orc_att_one_v5_f16(const orc_half *x, const orc_half *sx, float *s, const orc_half *ln_w,
                        const orc_half *ln_b, const float *lx_w, const float *lx_b,
                        const orc_half *k_mix, const orc_half *v_mix, const orc_half *r_mix,
                        const float *t_decay, const float *t_first, const orc_half *kw,
                        const orc_half *vw, const orc_half *rw, const orc_half *ow,
                        orc_half *x_out, orc_half *xx_out, int C, int H) {
  att_v5_0_f16(x, sx, s, ln_w, ln_b, lx_w, lx_b, k_mix, v_mix, r_mix, t_decay, t_first, kw, vw, rw,
               ow, x_out, xx_out, 1, C, H, 0);
}

void orc_att_seq_v5_f16(const orc_half *x, const orc_half *sx, float *s, const orc_half *ln_w,
                        const orc_half *ln_b, const float *lx_w, const float *lx_b,
                        const orc_half *k_mix, const orc_half *v_mix, const orc_half *r_mix,
                        const float *t_decay, const float *t_first, const orc_half *kw,
                        const orc_half *vw, const orc_half *rw, const orc_half *ow,
                        orc_half *x_out, orc_half *xx_last_out, int T, int C, int H) {
  att_v5_0_f16(x, sx, s, ln_w, ln_b, lx_w, lx_b, k_mix, v_mix, r_mix, t_decay, t_first, kw, vw, rw,
               ow, x_out, xx_last_out, T, C, H, 1);
}

/* ======================================================================== */
/* layer-level ops, fp32 (kernels/default/att.cpp, ffn.cpp)                  */
/* ======================================================================== */

static void att_one_v4_f32(const float *x, float *sx, float *aa, float *bb, float *pp,
                           const float *const *p, float *x_out, int C) {
  /* p: ln_w ln_b k_mix v_mix r_mix t_decay t_first kw vw rw ow  (att.cpp:16-45) */
  float *xx = (float *)xmalloc(4 * (size_t)C), *kx = (float *)xmalloc(4 * (size_t)C);
  float *vx = (float *)xmalloc(4 * (size_t)C), *rx = (float *)xmalloc(4 * (size_t)C);
  float *k = (float *)xmalloc(4 * (size_t)C), *v = (float *)xmalloc(4 * (size_t)C);
  float *r = (float *)xmalloc(4 * (size_t)C), *out = (float *)xmalloc(4 * (size_t)C);
  orc_layernorm_f32(x, p[0], p[1], xx, 1, C);
  orc_mix_f32(xx, sx, p[2], kx, 1, C);
  orc_mix_f32(xx, sx, p[3], vx, 1, C);
  orc_mix_f32(xx, sx, p[4], rx, 1, C);
  orc_gemm_f32(rx, p[9], r, 1, C, C);
  for (int i = 0; i < C; i++) r[i] = 1.0f / (1.0f + expf(-r[i]));
  orc_gemm_f32(kx, p[7], k, 1, C, C);
  orc_gemm_f32(vx, p[8], v, 1, C, C);
  wkv4_one_f32(p[6], p[5], k, v, aa, bb, pp, r, C);
  orc_gemm_f32(r, p[10], out, 1, C, C);
  for (int i = 0; i < C; i++) x_out[i] = x[i] + out[i];
  memcpy(sx, xx, 4 * (size_t)C);
  free(xx); free(kx); free(vx); free(rx); free(k); free(v); free(r); free(out);
}

static void ffn_one_f32(const float *x, float *sx, const float *const *p, float *x_out, int C,
                        int F) {
  /* p: ln_w ln_b k_mix r_mix kw vw rw  (ffn.cpp:8-23) */
  float *xx = (float *)xmalloc(4 * (size_t)C), *kx = (float *)xmalloc(4 * (size_t)C);
  float *rx = (float *)xmalloc(4 * (size_t)C), *r = (float *)xmalloc(4 * (size_t)C);
  float *vx = (float *)xmalloc(4 * (size_t)F), *out = (float *)xmalloc(4 * (size_t)C);
  orc_layernorm_f32(x, p[0], p[1], xx, 1, C);
  orc_mix_f32(xx, sx, p[2], kx, 1, C);
  orc_mix_f32(xx, sx, p[3], rx, 1, C);
  orc_gemm_f32(rx, p[6], r, 1, C, C);
  for (int i = 0; i < C; i++) r[i] = 1.0f / (1.0f + expf(-r[i]));
  orc_gemm_f32(kx, p[4], vx, 1, C, F);
  for (int i = 0; i < F; i++) {
    float t = vx[i] > 0.f ? vx[i] : 0.f;
    vx[i] = t * t;
  }
  orc_gemm_f32(vx, p[5], out, 1, F, C);
  for (int i = 0; i < C; i++) x_out[i] = x[i] + r[i] * out[i];
  memcpy(sx, xx, 4 * (size_t)C);
  free(xx); free(kx); free(rx); free(r); free(vx); free(out);
}

static void att_one_v5_2_f32(const float *x, float *sx, float *s, const float *const *p,
                             float *x_out, int C, int H) {
  /* p: ln_w ln_b lx_w lx_b k_mix v_mix r_mix g_mix t_decay t_first kw vw rw gw ow
   * (att.cpp:80-113, gate taken from gx as kernels/cuda/att.cu:289 does) */
  int S = C / H;
  size_t c = (size_t)C;
  float *xx = (float *)xmalloc(4 * c), *kx = (float *)xmalloc(4 * c), *vx = (float *)xmalloc(4 * c);
  float *rx = (float *)xmalloc(4 * c), *gx = (float *)xmalloc(4 * c), *k = (float *)xmalloc(4 * c);
  float *v = (float *)xmalloc(4 * c), *r = (float *)xmalloc(4 * c), *g = (float *)xmalloc(4 * c);
  float *y = (float *)xmalloc(4 * c), *gn = (float *)xmalloc(4 * c), *out = (float *)xmalloc(4 * c);
  orc_layernorm_f32(x, p[0], p[1], xx, 1, C);
  orc_mix_f32(xx, sx, p[4], kx, 1, C);
  orc_mix_f32(xx, sx, p[5], vx, 1, C);
  orc_mix_f32(xx, sx, p[6], rx, 1, C);
  orc_mix_f32(xx, sx, p[7], gx, 1, C);
  orc_gemm_f32(rx, p[12], r, 1, C, C);
  orc_gemm_f32(kx, p[10], k, 1, C, C);
  orc_gemm_f32(vx, p[11], v, 1, C, C);
  orc_gemm_f32(gx, p[13], g, 1, C, C);
  for (int i = 0; i < C; i++) g[i] = g[i] / (1.0f + expf(-g[i]));
  wkv5_one_f32(s, r, k, v, p[8], p[9], y, H, S);
  orc_groupnorm_f32(y, H, p[2], p[3], gn, 1, C);
  for (int i = 0; i < C; i++) gn[i] *= g[i];
  orc_gemm_f32(gn, p[14], out, 1, C, C);
  for (int i = 0; i < C; i++) x_out[i] = x[i] + out[i];
  memcpy(sx, xx, 4 * c);
  free(xx); free(kx); free(vx); free(rx); free(gx); free(k); free(v); free(r); free(g); free(y); free(gn); free(out);
}

/* ======================================================================== */
/* whole model                                                               */
/* ======================================================================== */

static int per_layer_states(const orc_model *m) { return m->version == 4 ? 5 : 3; }

size_t orc_state_count(const orc_model *m) { return (size_t)m->n_layer * per_layer_states(m); }

int orc_state_is_act(const orc_model *m, size_t idx) {
  int j = (int)(idx % per_layer_states(m));
  return m->version == 4 ? (j == 0 || j == 4) : (j == 0 || j == 2);
}

size_t orc_state_elems(const orc_model *m, size_t idx) {
  int j = (int)(idx % per_layer_states(m));
  if (m->version == 4) return (j == 0 || j == 4) ? (size_t)m->n_embd : (size_t)m->n_att;
  if (j == 1) { /* model.cpp:169-171: [n_head, n_att/n_head, n_embd/n_head] */
    return (size_t)m->n_head * (m->n_att / m->n_head) * (m->n_embd / m->n_head);
  }
  return (size_t)m->n_embd;
}

void orc_state_reset(const orc_model *m, void *const *state) {
  size_t cnt = orc_state_count(m);
  for (size_t i = 0; i < cnt; i++) {
    size_t n = orc_state_elems(m, i);
    int j = (int)(i % per_layer_states(m));
    if (orc_state_is_act(m, i)) {
      memset(state[i], 0, n * (m->mode == ORC_F16 ? 2 : 4));
    } else {
      float *f = (float *)state[i];
      float val = (m->version == 4 && j == 3) ? -1e30f : 0.f; /* model.cpp:158-159 */
      for (size_t e = 0; e < n; e++) f[e] = val;
    }
  }
}

int orc_argmax(const float *x, int n) {
  int best = 0;
  for (int i = 1; i < n; i++)
    if (x[i] > x[best]) best = i;
  return best;
}

static void forward_seq_f16(const orc_model *m, void *const *state, const int *ids, int T,
                            float *logits) {
  int C = m->n_embd, F = m->n_ffn, V = m->vocab;
  size_t n = (size_t)T * C;
  orc_half *x = (orc_half *)xmalloc(2 * n), *y = (orc_half *)xmalloc(2 * n);
  const orc_half *emb = (const orc_half *)m->emb;
  for (int t = 0; t < T; t++) memcpy(x + (size_t)t * C, emb + (size_t)ids[t] * C, 2 * (size_t)C);
  const void *const *p = m->params;
  const orc_half two = 0x4000;
  orc_half *xx_last = (orc_half *)xmalloc(2 * (size_t)C);
  for (int l = 0; l < m->n_layer; l++) {
    void *const *st = state + (size_t)l * per_layer_states(m);
    if (m->version == 4) {
      orc_att_seq_v4_f16(x, (const orc_half *)st[0], (float *)st[1], (float *)st[2], (float *)st[3],
                         (const orc_half *)p[0], (const orc_half *)p[1], (const orc_half *)p[2],
                         (const orc_half *)p[3], (const orc_half *)p[4], (const float *)p[5],
                         (const float *)p[6], (const orc_half *)p[7], (const orc_half *)p[8],
                         (const orc_half *)p[9], (const orc_half *)p[10], y, xx_last, T, C);
      memcpy(st[0], xx_last, 2 * (size_t)C);
      p += 11;
      orc_ffn_seq_f16(y, (const orc_half *)st[4], (const orc_half *)p[0], (const orc_half *)p[1],
                      (const orc_half *)p[2], (const orc_half *)p[3], (const orc_half *)p[4],
                      (const orc_half *)p[5], (const orc_half *)p[6], x, xx_last, T, C, F);
      memcpy(st[4], xx_last, 2 * (size_t)C);
      p += 7;
    } else if (m->version == 50) { /* model_forward.cpp:124-137, model_forward_seq.cpp:113-126 */
      att_v5_0_f16(x, (const orc_half *)st[0], (float *)st[1], (const orc_half *)p[0],
                   (const orc_half *)p[1], (const float *)p[2], (const float *)p[3],
                   (const orc_half *)p[4], (const orc_half *)p[5], (const orc_half *)p[6],
                   (const float *)p[7], (const float *)p[8], (const orc_half *)p[9],
                   (const orc_half *)p[10], (const orc_half *)p[11], (const orc_half *)p[12], y,
                   xx_last, T, C, m->n_head, T > 1);
      memcpy(st[0], xx_last, 2 * (size_t)C);
      p += 13;
      orc_ffn_seq_f16(y, (const orc_half *)st[2], (const orc_half *)p[0], (const orc_half *)p[1],
                      (const orc_half *)p[2], (const orc_half *)p[3], (const orc_half *)p[4],
                      (const orc_half *)p[5], (const orc_half *)p[6], x, xx_last, T, C, F);
      memcpy(st[2], xx_last, 2 * (size_t)C);
      p += 7;
    } else {
      att_v5_2_f16(x, (const orc_half *)st[0], (float *)st[1], (const orc_half *)p[0],
                   (const orc_half *)p[1], (const float *)p[2], (const float *)p[3],
                   (const orc_half *)p[4], (const orc_half *)p[5], (const orc_half *)p[6],
                   (const orc_half *)p[7], (const float *)p[8], (const float *)p[9],
                   (const orc_half *)p[10], (const orc_half *)p[11], (const orc_half *)p[12],
                   (const orc_half *)p[13], (const orc_half *)p[14], y, xx_last, T, C, m->n_head,
                   T > 1 /* seq mode uses the scan kernel's form, one mode the functor's */);
      memcpy(st[0], xx_last, 2 * (size_t)C);
      p += 15;
      orc_ffn_seq_f16(y, (const orc_half *)st[2], (const orc_half *)p[0], (const orc_half *)p[1],
                      (const orc_half *)p[2], (const orc_half *)p[3], (const orc_half *)p[4],
                      (const orc_half *)p[5], (const orc_half *)p[6], x, xx_last, T, C, F);
      memcpy(st[2], xx_last, 2 * (size_t)C);
      p += 7;
    }
    if ((l + 1) % 6 == 0) /* model_forward.cpp:173-175 */
      for (size_t i = 0; i < n; i++) x[i] = orc_hdiv(x[i], two);
  }
  orc_half *last = x + (size_t)(T - 1) * C; /* model_forward_seq.cpp:170-172 */
  orc_half *ln = (orc_half *)xmalloc(2 * (size_t)C), *lg = (orc_half *)xmalloc(2 * (size_t)V);
  orc_layernorm_f16(last, (const orc_half *)p[0], (const orc_half *)p[1], ln, 1, C);
  orc_gemm_f16(ln, (const orc_half *)p[2], NULL, lg, 1, C, V);
  orc_h2f_n(lg, logits, (size_t)V);
  free(x); free(y); free(xx_last); free(ln); free(lg);
}

static void forward_one_f32(const orc_model *m, void *const *state, int id, float *logits) {
  int C = m->n_embd, F = m->n_ffn, V = m->vocab;
  float *x = (float *)xmalloc(4 * (size_t)C), *y = (float *)xmalloc(4 * (size_t)C);
  memcpy(x, (const float *)m->emb + (size_t)id * C, 4 * (size_t)C);
  const float *const *p = (const float *const *)m->params;
  for (int l = 0; l < m->n_layer; l++) {
    void *const *st = state + (size_t)l * per_layer_states(m);
    if (m->version == 4) {
      att_one_v4_f32(x, (float *)st[0], (float *)st[1], (float *)st[2], (float *)st[3], p, y, C);
      p += 11;
      ffn_one_f32(y, (float *)st[4], p, x, C, F);
      p += 7;
    } else if (m->version == 50) {
      fprintf(stderr, "rwkv_oracle: RWKV-5.0 is restated in ORC_F16 mode only\n");
      abort();
    } else {
      att_one_v5_2_f32(x, (float *)st[0], (float *)st[1], p, y, C, m->n_head);
      p += 15;
      ffn_one_f32(y, (float *)st[2], p, x, C, F);
      p += 7;
    }
    /* no /2 rescale: model_forward.cpp:173 applies it to fp16 activations only */
  }
  orc_layernorm_f32(x, p[0], p[1], y, 1, C);
  orc_gemm_f32(y, p[2], logits, 1, C, V);
  free(x); free(y);
}

void orc_model_forward(const orc_model *m, void *const *state, int id, float *logits) {
  if (m->mode == ORC_F16)
    forward_seq_f16(m, state, &id, 1, logits);
  else
    forward_one_f32(m, state, id, logits);
}

void orc_model_forward_seq(const orc_model *m, void *const *state, const int *ids, int T,
                           float *logits) {
  if (m->mode == ORC_F16) {
    forward_seq_f16(m, state, ids, T, logits);
  } else { /* model_forward_seq.cpp:34-46 */
    for (int t = 0; t < T; t++) forward_one_f32(m, state, ids[t], logits);
  }
}
