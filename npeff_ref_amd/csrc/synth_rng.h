/*
 * Counter-based random numbers and the synthetic-PEF sampler, written so that
 * the host (gcc) and the device (hipcc, gfx950) produce the same bits: only
 * IEEE add/mul/div/sqrt/fma on doubles and integer arithmetic, no libm.  Both
 * builds compile this header with -ffp-contract=off; every fused operation is
 * an explicit fma().
 *
 * This stands in for curandGenerateUniform (XORWOW), whose stream cannot be
 * reproduced without cuRAND
 * (cc/cuda_d_npeff/src/nmf/sparse/multi_mu_dense_factors_device_contexts1.h:197-207):
 * factors are U[0,1) values keyed by (seed, matrix, logical element).
 */
#ifndef DNPEFF_SYNTH_RNG_H_
#define DNPEFF_SYNTH_RNG_H_

#include <stdint.h>
#if !defined(__HIPCC__)
#include <math.h>
#endif

#if defined(__HIPCC__)
#define DN_HD __host__ __device__ inline
#else
#define DN_HD static inline
#endif

#define DN_TAG_INIT 0x1f83d9abfb41bd6bULL
#define DN_TAG_ZIPF 0x5be0cd19137e2179ULL
#define DN_TAG_VAL 0x3c6ef372fe94f82bULL
#define DN_TAG_LEN 0xa54ff53a5f1d36f1ULL

DN_HD uint64_t dn_mix64(uint64_t x) {
  x ^= x >> 30;
  x *= 0xbf58476d1ce4e5b9ULL;
  x ^= x >> 27;
  x *= 0x94d049bb133111ebULL;
  x ^= x >> 31;
  return x;
}

/* Hash of (seed, a, b): two rounds of the splitmix64 finaliser. */
DN_HD uint64_t dn_hash3(uint64_t seed, uint64_t a, uint64_t b) {
  uint64_t x = dn_mix64(seed + 0x9e3779b97f4a7c15ULL * (a + 1));
  x = dn_mix64(x ^ (0xd1b54a32d192ed03ULL * (b + 1)));
  return x;
}

/* 24 random bits -> [0, 1) in fp32, exactly representable. */
DN_HD float dn_u01f(uint64_t h) { return (float)(h >> 40) * (1.0f / 16777216.0f); }

/* 52 random bits -> (0, 1) in fp64, never 0 or 1. */
DN_HD double dn_u01d(uint64_t h) {
  return ((double)(h >> 12) + 0.5) * (1.0 / 4503599627370496.0);
}

DN_HD float dn_uniform_at(uint64_t seed, int matrix_id, int64_t row, int64_t col, int64_t n_cols) {
  uint64_t idx = (uint64_t)row * (uint64_t)n_cols + (uint64_t)col;
  return dn_u01f(dn_hash3(seed ^ DN_TAG_INIT, (uint64_t)matrix_id, idx));
}

/* ---- bit-reproducible elementary functions (double) ---- */

DN_HD uint64_t dn_d2u(double x) {
  union { double d; uint64_t u; } c;
  c.d = x;
  return c.u;
}
DN_HD double dn_u2d(uint64_t u) {
  union { double d; uint64_t u; } c;
  c.u = u;
  return c.d;
}

/* Natural log of a positive, finite, normal double. */
DN_HD double dn_log(double x) {
  uint64_t u = dn_d2u(x);
  int64_t e = (int64_t)((u >> 52) & 0x7ff) - 1023;
  double m = dn_u2d((u & 0x000fffffffffffffULL) | 0x3ff0000000000000ULL); /* [1,2) */
  if (m > 1.4142135623730951) {
    m = m * 0.5;
    e += 1;
  }
  double f = (m - 1.0) / (m + 1.0); /* |f| <= 0.1716 */
  double f2 = f * f;
  /* 2*atanh(f) = 2 f (1 + f^2/3 + f^4/5 + ...), terms to f^24 */
  double p = 1.0 / 25.0;
  p = fma(p, f2, 1.0 / 23.0);
  p = fma(p, f2, 1.0 / 21.0);
  p = fma(p, f2, 1.0 / 19.0);
  p = fma(p, f2, 1.0 / 17.0);
  p = fma(p, f2, 1.0 / 15.0);
  p = fma(p, f2, 1.0 / 13.0);
  p = fma(p, f2, 1.0 / 11.0);
  p = fma(p, f2, 1.0 / 9.0);
  p = fma(p, f2, 1.0 / 7.0);
  p = fma(p, f2, 1.0 / 5.0);
  p = fma(p, f2, 1.0 / 3.0);
  p = fma(p, f2, 1.0);
  double lm = 2.0 * f * p;
  return fma((double)e, 0.6931471805599453, lm);
}

/* exp(x) for |x| < 700. */
DN_HD double dn_exp(double x) {
  double kf = x * 1.4426950408889634;
  int64_t k = (int64_t)(kf + (kf >= 0.0 ? 0.5 : -0.5));
  double r = fma(-(double)k, 0.6931471803691238, x);   /* ln2 high part */
  r = fma(-(double)k, 1.9082149292705877e-10, r);      /* ln2 low part  */
  double p = 1.0 / 87178291200.0; /* 1/14! */
  p = fma(p, r, 1.0 / 6227020800.0);
  p = fma(p, r, 1.0 / 479001600.0);
  p = fma(p, r, 1.0 / 39916800.0);
  p = fma(p, r, 1.0 / 3628800.0);
  p = fma(p, r, 1.0 / 362880.0);
  p = fma(p, r, 1.0 / 40320.0);
  p = fma(p, r, 1.0 / 5040.0);
  p = fma(p, r, 1.0 / 720.0);
  p = fma(p, r, 1.0 / 120.0);
  p = fma(p, r, 1.0 / 24.0);
  p = fma(p, r, 1.0 / 6.0);
  p = fma(p, r, 0.5);
  p = fma(p, r, 1.0);
  p = fma(p, r, 1.0);
  /* scale by 2^k through the exponent field (k in [-1010, 1010]) */
  return p * dn_u2d((uint64_t)(k + 1023) << 52);
}

/* Standard normal from a uniform in (0,1): Acklam's rational inverse CDF
 * (relative error < 1.2e-9, ample for synthetic values). */
DN_HD double dn_norm_inv(double p) {
  const double a0 = -3.969683028665376e+01, a1 = 2.209460984245205e+02,
               a2 = -2.759285104469687e+02, a3 = 1.383577518672690e+02,
               a4 = -3.066479806614716e+01, a5 = 2.506628277459239e+00;
  const double b0 = -5.447609879822406e+01, b1 = 1.615858368580409e+02,
               b2 = -1.556989798598866e+02, b3 = 6.680131188771972e+01,
               b4 = -1.328068155288572e+01;
  const double c0 = -7.784894002430293e-03, c1 = -3.223964580411365e-01,
               c2 = -2.400758277161838e+00, c3 = -2.549732539343734e+00,
               c4 = 4.374664141464968e+00, c5 = 2.938163982698783e+00;
  const double d0 = 7.784695709041462e-03, d1 = 3.224671290700398e-01,
               d2 = 2.445134137142996e+00, d3 = 3.754408661907416e+00;
  const double plow = 0.02425;
  if (p < plow) {
    double q = sqrt(-2.0 * dn_log(p));
    double num = fma(fma(fma(fma(fma(c0, q, c1), q, c2), q, c3), q, c4), q, c5);
    double den = fma(fma(fma(fma(d0, q, d1), q, d2), q, d3), q, 1.0);
    return num / den;
  }
  if (p > 1.0 - plow) {
    double q = sqrt(-2.0 * dn_log(1.0 - p));
    double num = fma(fma(fma(fma(fma(c0, q, c1), q, c2), q, c3), q, c4), q, c5);
    double den = fma(fma(fma(fma(d0, q, d1), q, d2), q, d3), q, 1.0);
    return -(num / den);
  }
  double q = p - 0.5;
  double r = q * q;
  double num = fma(fma(fma(fma(fma(a0, r, a1), r, a2), r, a3), r, a4), r, a5) * q;
  double den = fma(fma(fma(fma(fma(b0, r, b1), r, b2), r, b3), r, b4), r, 1.0);
  return num / den;
}

/* ---- Zipf(s) over {1..N}, s != 1, by rejection-inversion
 * (Hormann & Derflinger 1996) ---- */

typedef struct {
  double s;         /* exponent */
  double oms;       /* 1 - s */
  double n;         /* number of elements */
  double h_x1;      /* H(1.5) - 1 */
  double h_n;       /* H(N + 0.5) */
  double accept_s;  /* 2 - Hinv(H(2.5) - h(2)) */
} dn_zipf;

DN_HD double dn_zipf_H(const dn_zipf* z, double x) {
  return (dn_exp(z->oms * dn_log(x)) - 1.0) / z->oms;
}
DN_HD double dn_zipf_h(const dn_zipf* z, double x) { return dn_exp(-z->s * dn_log(x)); }
DN_HD double dn_zipf_Hinv(const dn_zipf* z, double x) {
  double t = x * z->oms;
  if (t < -1.0 + 1e-15) t = -1.0 + 1e-15;
  return dn_exp(dn_log(1.0 + t) / z->oms);
}

DN_HD void dn_zipf_init(dn_zipf* z, double s, int64_t n) {
  z->s = s;
  z->oms = 1.0 - s;
  z->n = (double)n;
  z->h_x1 = dn_zipf_H(z, 1.5) - 1.0;
  z->h_n = dn_zipf_H(z, (double)n + 0.5);
  z->accept_s = 2.0 - dn_zipf_Hinv(z, dn_zipf_H(z, 2.5) - dn_zipf_h(z, 2.0));
}

/* Draw number t of row `row`: a rank in [0, N) (rank 1 <-> id 0).  Each
 * rejection attempt consumes one keyed uniform; at most 16 attempts. */
DN_HD int64_t dn_zipf_draw(const dn_zipf* z, uint64_t seed, uint64_t row, uint64_t t) {
  int64_t k = 1;
  for (uint64_t a = 0; a < 16; a++) {
    double u01 = dn_u01d(dn_hash3(seed ^ DN_TAG_ZIPF, row, t * 16 + a));
    double u = fma(u01, z->h_x1 - z->h_n, z->h_n);
    double x = dn_zipf_Hinv(z, u);
    k = (int64_t)(x + 0.5);
    if (k < 1) k = 1;
    if ((double)k > z->n) k = (int64_t)z->n;
    if ((double)k - x <= z->accept_s) break;
    if (u >= dn_zipf_H(z, (double)k + 0.5) - dn_zipf_h(z, (double)k)) break;
  }
  return k - 1;
}

/* Entry value number p of row `row`: exp(N(mu, sigma^2)) rounded to fp32. */
DN_HD float dn_lognormal_at(uint64_t seed, uint64_t row, uint64_t p, double mu, double sigma) {
  double u = dn_u01d(dn_hash3(seed ^ DN_TAG_VAL, row, p));
  double zn = dn_norm_inv(u);
  return (float)dn_exp(fma(sigma, zn, mu));
}

/* Row length: k_fixed, or round(exp(U(ln k_min, ln k_max))) when k_min > 0. */
DN_HD int64_t dn_row_length(uint64_t seed, uint64_t row, int64_t k_fixed, int64_t k_min,
                            int64_t k_max) {
  if (k_min <= 0) return k_fixed;
  double u = dn_u01d(dn_hash3(seed ^ DN_TAG_LEN, row, 0));
  double lo = dn_log((double)k_min), hi = dn_log((double)k_max);
  double v = dn_exp(fma(u, hi - lo, lo));
  int64_t k = (int64_t)(v + 0.5);
  if (k < k_min) k = k_min;
  if (k > k_max) k = k_max;
  return k;
}

#endif /* DNPEFF_SYNTH_RNG_H_ */
