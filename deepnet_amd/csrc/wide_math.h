// Transcendentals for fp32 inputs evaluated with fp64 internals to a relative
// error of about 2^-33, so that a whole formula (exp -> add -> divide, log of a
// sum, a * cos(b) ...) is rounded to fp32 once, at its end.  The fp32 library
// routines are each allowed a few ulp and a chain of them drifts past the
// 2-ulp parity bar.  fp64 instructions issue at half the fp32 rate, which a
// streaming kernel mostly hides; exp and sigmoid, the two that showed it, have
// fp32 routes of about 1 ulp for arguments of ordinary size.
#pragma once
#include <hip/hip_runtime.h>
#include <math.h>

// 1/d for finite non-zero d: hardware estimate plus one Newton step.
__device__ __forceinline__ double dn_rcp_wide(double d) {
  double r = __builtin_amdgcn_rcp(d);
  return r * fma(-d, r, 2.0);
}

// e^t and e^t - 1.  t*log2(e) is split into an integer n and a fraction; with
// g = fraction*ln2, |g| <= 0.347, q(g) = e^g - 1 is a degree-8 Taylor sum
// (remainder g^9/9! < 2.1e-10 of e^g).  e^t = 2^n (1 + q); e^t - 1 is q itself
// when n == 0, which keeps full relative accuracy for small t.  Arguments beyond
// +-800 saturate (0 or inf in fp64 either way).
__device__ __forceinline__ double dn_exp_parts(double t, double* n_out) {
  t = fmin(fmax(t, -800.0), 800.0) * 1.4426950408889634;
  const double n = rint(t);
  const double g = (t - n) * 0.6931471805599453;
  double p = 2.48015873015873e-05;       // 1/8!
  p = fma(p, g, 1.984126984126984e-04);  // 1/7!
  p = fma(p, g, 1.388888888888889e-03);  // 1/6!
  p = fma(p, g, 8.333333333333333e-03);  // 1/5!
  p = fma(p, g, 4.166666666666666e-02);  // 1/4!
  p = fma(p, g, 1.666666666666667e-01);  // 1/3!
  p = fma(p, g, 0.5);
  p = fma(p, g, 1.0);
  *n_out = n;
  return p * g;  // q(g)
}
__device__ __forceinline__ double dn_exp_wide(double t) {
  double n;
  const double q = dn_exp_parts(t, &n);
  return ldexp(1.0 + q, (int)n);
}
__device__ __forceinline__ double dn_expm1_wide(double t) {
  double n;
  const double q = dn_exp_parts(t, &n);
  return n == 0.0 ? q : ldexp(1.0 + q, (int)n) - 1.0;
}

// ln(x) for finite x > 0 (callers handle 0, negatives, inf, NaN).
// x = m * 2^e with m in [sqrt(1/2), sqrt(2)); ln m = 2*atanh(s), s = (m-1)/(m+1),
// |s| <= 0.1716, series through s^12/13 (remainder below 2^-39 of the result).
__device__ __forceinline__ double dn_log_wide_pos(double x) {
  int e;
  double m = frexp(x, &e);  // m in [0.5, 1)
  if (m < 0.7071067811865476) { m *= 2.0; e -= 1; }
  const double s = (m - 1.0) * dn_rcp_wide(m + 1.0);
  const double z = s * s;
  double p = 1.0 / 13.0;
  p = fma(p, z, 1.0 / 11.0);
  p = fma(p, z, 1.0 / 9.0);
  p = fma(p, z, 1.0 / 7.0);
  p = fma(p, z, 1.0 / 5.0);
  p = fma(p, z, 1.0 / 3.0);
  p = fma(p, z, 1.0);
  return fma((double)e, 0.6931471805599453, 2.0 * s * p);
}

// ln(x) with logf's special values, still in fp64.
__device__ __forceinline__ double dn_log_wide(float x) {
  if (x > 0.f && x < INFINITY) return dn_log_wide_pos((double)x);
  if (x == 0.f) return -(double)INFINITY;
  if (x < 0.f) return (double)NAN;
  return (double)x;  // +inf or NaN
}
__device__ __forceinline__ float dn_log(float x) { return (float)dn_log_wide(x); }

// ln(1 + e^x): x + ln(1 + e^-x) for x > 0, ln(1 + e^x) otherwise; ln(1 + u) for a
// tiny u is u - u^2/2 + u^3/3 (1 + u itself would round u away).
__device__ __forceinline__ float dn_softplus(float x) {
  if (x != x) return x;
  const double u = dn_exp_wide(-(double)fabsf(x));  // in (0, 1]
  const double l = u < 1e-5 ? u * fma(u, fma(u, 1.0 / 3.0, -0.5), 1.0) : dn_log_wide_pos(1.0 + u);
  return (float)(x > 0.f ? l + (double)x : l);
}

// The same split in fp32 for arguments of ordinary size (fp64 instructions issue at half the
// fp32 rate here, and exp / sigmoid over a large matrix are otherwise issue-bound):
// n = rint(t log2 e), g = t - n ln2 in two FMAs (the first is exact: n has at most 8 significant
// bits, the high part of ln2 has 16), e^g - 1 = g + g^2 P(g) with P the Taylor sum through g^5
// (remainder g^8/8! < 5.2e-9).  Returns e^g - 1 to about half an ulp of e^g.
__device__ __forceinline__ float dn_exp_parts_f32(float t, float* n_out) {
  const float n = rintf(t * 1.44269504088896341f);
  float g = fmaf(n, -0.693145751953125f, t);
  g = fmaf(n, -1.42860682030941723e-06f, g);
  float p = 1.98412698412698413e-04f;      // 1/7!
  p = fmaf(p, g, 1.38888888888888894e-03f);  // 1/6!
  p = fmaf(p, g, 8.33333333333333322e-03f);  // 1/5!
  p = fmaf(p, g, 4.16666666666666644e-02f);  // 1/4!
  p = fmaf(p, g, 1.66666666666666657e-01f);  // 1/3!
  p = fmaf(p, g, 0.5f);
  *n_out = n;
  return fmaf(g * g, p, g);
}

// e^x: one rounding of 1 + (e^g - 1) and an exact scaling for |x| <= 80 (results between
// 1.8e-35 and 5.5e34: about 1 ulp in all); the fp64 evaluation beyond, and for NaN.
__device__ __forceinline__ float dn_exp(float x) {
  if (fabsf(x) <= 80.f) {
    float n;
    const float q = dn_exp_parts_f32(x, &n);
    return ldexpf(1.0f + q, (int)n);
  }
  return x != x ? x : (float)dn_exp_wide((double)x);
}

// 1/(1+exp(-x)).  For |x| <= 16: e^-x = 2^n (1 + q) with |n| <= 23, so the sum 1 + 2^n is
// exact, s = 2^n q + (1 + 2^n) is rounded once and the rounding error kept (a result just
// below a power of two would double it), and the reciprocal of the pair is the hardware
// estimate with one Newton step (about 1 ulp in all).
// The fp64 evaluation beyond, and for NaN.
__device__ __forceinline__ float dn_sigmoid(float x) {
  if (fabsf(x) <= 16.f) {
    float n;
    const float q = dn_exp_parts_f32(-x, &n);
    const float p2 = ldexpf(1.0f, (int)n);
    const float hi = 1.0f + p2;
    const float s = fmaf(p2, q, hi);
    const float s_lo = fmaf(p2, q, hi - s);          // what the rounding of s dropped (hi - s is exact)
    const float r = __builtin_amdgcn_rcpf(s);
    return fmaf(r, fmaf(-s_lo, r, fmaf(-s, r, 1.0f)), r);
  }
  const double s = 1.0 + dn_exp_wide(-(double)x);   // in [1, inf]
  const float r = (s < 1e300) ? (float)dn_rcp_wide(s) : 0.f;
  return x != x ? x : r;
}

// tanh(x), the value of the reference's formula 1 - 2/(e^2x + 1), in fp32 (measured <= 0.9 ulp).
// |x| <= 0.625: x + x^3 P(x^2), P a degree-5 fit of (tanh(x)/x - 1)/x^2 at Chebyshev nodes
// (error 2e-10 of tanh).  Beyond: e^2|x| = 2^n (1 + q), the denominator 2^n q + (2^n + 1) with
// its rounding error kept, its reciprocal by the hardware estimate and one Newton step, and
// one more rounding in 1 - 2r; from |x| = 9.02 on that is 1.
__device__ __forceinline__ float dn_tanh(float x) {
  const float ax = fabsf(x);
  if (ax <= 0.625f) {
    const float z = ax * ax;
    float p = 0.002292744815349579f;
    p = fmaf(p, z, -0.008343945257365704f);
    p = fmaf(p, z, 0.02176891826093197f);
    p = fmaf(p, z, -0.053959257900714874f);
    p = fmaf(p, z, 0.13333304226398468f);
    p = fmaf(p, z, -0.3333333432674408f);
    return copysignf(fmaf(ax * z, p, ax), x);
  }
  if (x != x) return x;
  float n;
  const float q = dn_exp_parts_f32(2.f * fminf(ax, 20.f), &n);
  const float p2 = ldexpf(1.0f, (int)n);
  const float hi = p2 + 1.0f;
  const float d = fmaf(p2, q, hi);
  const float d_lo = fmaf(p2, q, hi - d);
  const float r = __builtin_amdgcn_rcpf(d);
  const float r1 = fmaf(r, fmaf(-d_lo, r, fmaf(-d, r, 1.0f)), r);
  return copysignf(fmaf(-2.f, r1, 1.0f), x);
}

// sin and cos of x.  Cody-Waite reduction by pi/2 in fp64 (exact through the FMA
// for |x| < 2^30), then Taylor sums on [-pi/4, pi/4] (remainders < 1e-11).
// Larger arguments take the library's fp64 routines.
__device__ __forceinline__ void dn_sincos_wide(float x, double* sn, double* cs) {
  const double xd = (double)x;
  if (!(fabsf(x) < 1.0e9f)) {  // huge, inf or NaN
    *sn = sin(xd);
    *cs = cos(xd);
    return;
  }
  const double k = rint(xd * 0.6366197723675814);
  double r = fma(-k, 1.5707963267948966, xd);
  r = fma(-k, 6.123233995736766e-17, r);
  const double z = r * r;
  double ps = -2.505210838544172e-08;      // -1/11!
  ps = fma(ps, z, 2.755731922398589e-06);  //  1/9!
  ps = fma(ps, z, -1.984126984126984e-04); // -1/7!
  ps = fma(ps, z, 8.333333333333333e-03);  //  1/5!
  ps = fma(ps, z, -1.666666666666667e-01); // -1/3!
  const double s = fma(r * z, ps, r);
  double pc = 2.08767569878681e-09;        //  1/12!
  pc = fma(pc, z, -2.755731922398589e-07); // -1/10!
  pc = fma(pc, z, 2.48015873015873e-05);   //  1/8!
  pc = fma(pc, z, -1.388888888888889e-03); // -1/6!
  pc = fma(pc, z, 4.166666666666666e-02);  //  1/4!
  pc = fma(pc, z, -0.5);
  const double c = fma(pc, z, 1.0);
  const int q = (int)k & 3;
  const double s_out = (q & 1) ? c : s;
  const double c_out = (q & 1) ? s : c;
  *sn = (q & 2) ? -s_out : s_out;
  *cs = ((q + 1) & 2) ? -c_out : c_out;
}
__device__ __forceinline__ double dn_sin_wide(float x) { double s, c; dn_sincos_wide(x, &s, &c); return s; }
__device__ __forceinline__ double dn_cos_wide(float x) { double s, c; dn_sincos_wide(x, &s, &c); return c; }

// powf(x, p) as exp(p * ln x) in fp64 for the ordinary cases (finite x != 0 with a
// finite p, negative x only with an integer p); everything else is an exact
// special value and is left to the library.
__device__ __forceinline__ float dn_pow(float x, float p) {
  const float ax = fabsf(x);
  const bool p_finite = fabsf(p) < INFINITY;
  if (ax > 0.f && ax < INFINITY && p_finite) {
    if (x > 0.f) return (float)dn_exp_wide((double)p * dn_log_wide_pos((double)ax));
    if (rintf(p) == p) {
      const float r = (float)dn_exp_wide((double)p * dn_log_wide_pos((double)ax));
      const bool odd = fabsf(p) < 16777216.f && (((long long)p) & 1);
      return odd ? -r : r;
    }
  }
  return powf(x, p);
}
