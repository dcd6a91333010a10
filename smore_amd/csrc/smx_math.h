// Device math for the distance functors: digamma, trigamma, log-gamma.
//
// Numerical contract: same series as the operator being replaced
// (smore/common/torchext/cuda_math_ext.h:130-211 -- reflection, upward
// recurrence, asymptotic tail), evaluated in the precision of T.
#pragma once
#include <hip/hip_runtime.h>

namespace smx {

template <typename T> struct MathConst;
template <> struct MathConst<float> {
  static constexpr float pi = 3.14159265358979323846f;
};
template <> struct MathConst<double> {
  static constexpr double pi = 3.14159265358979323846;
};

__device__ __forceinline__ float m_acc_log(float x) { return logf(x); }
__device__ __forceinline__ double m_acc_log(double x) { return log(x); }
__device__ __forceinline__ float m_sqrt(float x) { return sqrtf(x); }
__device__ __forceinline__ double m_sqrt(double x) { return sqrt(x); }
__device__ __forceinline__ float m_sin(float x) { return sinf(x); }
__device__ __forceinline__ double m_sin(double x) { return sin(x); }
__device__ __forceinline__ float m_lgamma(float x) { return lgammaf(x); }
__device__ __forceinline__ double m_lgamma(double x) { return lgamma(x); }
__device__ __forceinline__ float m_abs(float x) { return fabsf(x); }
__device__ __forceinline__ double m_abs(double x) { return fabs(x); }
__device__ __forceinline__ float m_min(float a, float b) { return fminf(a, b); }
__device__ __forceinline__ double m_min(double a, double b) { return fmin(a, b); }

// psi(x).  x == 0 -> -/+inf, negative integers -> NaN, x < 0 by reflection.
template <typename T>
__device__ inline T digamma(T x) {
  T shift = 0;
  if (x <= 0) {
    if (x == 0) return copysign((T)INFINITY, -x);
    if (x == trunc(x)) return (T)NAN;
    // the cotangent term is evaluated in double: rounding of pi*x matters near poles
    shift = (T)(-3.14159265358979323846 / tan(3.14159265358979323846 * (double)x));
    x = 1 - x;
  }
  while (x < 10) {
    shift -= 1 / x;
    x += 1;
  }
  if (x == 10) return shift + (T)2.25175258906672110764;
  T tail = 0;
  if (x < (T)1.0e17) {
    const T z = 1 / (x * x);
    T p = (T)8.33333333333333333333E-2;
    p = p * z + (T)-2.10927960927960927961E-2;
    p = p * z + (T)7.57575757575757575758E-3;
    p = p * z + (T)-4.16666666666666666667E-3;
    p = p * z + (T)3.96825396825396825397E-3;
    p = p * z + (T)-8.33333333333333333333E-3;
    p = p * z + (T)8.33333333333333333333E-2;
    tail = z * p;
  }
  return m_acc_log(x) - ((T)0.5 / x) - tail + shift;
}

// psi'(x).  x < 0.5 by reflection, six recurrence steps, asymptotic tail.
template <typename T>
__device__ inline T trigamma(T x) {
  const T pi = MathConst<T>::pi;
  T sign = 1, acc = 0;
  if (x < (T)0.5) {
    sign = -1;
    const T s = m_sin(pi * x);
    acc -= (pi * pi) / (s * s);
    x = 1 - x;
  }
#pragma unroll
  for (int i = 0; i < 6; ++i) {
    acc += 1 / (x * x);
    x += 1;
  }
  const T ixx = 1 / (x * x);
  acc += (1 + 1 / (2 * x) + ixx * ((T)1 / 6 - ixx * ((T)1 / 30 - ixx * ((T)1 / 42)))) / x;
  return sign * acc;
}

// ---- fast fp32 forms for the fused Beta-KL kernels ----------------------------------------------
// For fast_lo <= x <= fast_hi the argument is shifted by a fixed six steps, so there is no
// data-dependent loop and no division:
//   psi(x)    = psi(x+6)  - N(x)/D(x)            D(x) = x(x+1)...(x+5),  N = D'
//   psi'(x)   = psi'(x+6) + P10(x)/D(x)^2        P10 = N^2 - N' D (expanded: all coefficients positive)
//   lgamma(x) = lgamma(x+6) - ln D(x)
// with the asymptotic series at y = x+6 >= 6 (first neglected terms: 2.5e-9, 3.3e-9, 2.1e-9).  The
// polynomials have positive coefficients, so Horner's rule is free of cancellation for x > 0.
// Reciprocals and logarithms use the hardware approximations (1 ulp).  Outside the interval the
// callers fall back to the general routines above.
constexpr float kFastLo = 0.02f;
constexpr float kFastHi = 1000.0f;

__device__ __forceinline__ float f_rcp(float x) { return __builtin_amdgcn_rcpf(x); }
__device__ __forceinline__ float f_log(float x) { return __builtin_amdgcn_logf(x) * 0.69314718055994531f; }

__device__ __forceinline__ float poly_d6(float x) {
  return x * (120.f + x * (274.f + x * (225.f + x * (85.f + x * (15.f + x)))));
}
__device__ __forceinline__ float poly_n5(float x) {
  return 120.f + x * (548.f + x * (675.f + x * (340.f + x * (75.f + x * 6.f))));
}
__device__ __forceinline__ float poly_p10(float x) {
  return 14400.f + x * (65760.f + x * (150152.f + x * (205800.f + x * (180455.f + x * (104370.f + x * (40208.f +
         x * (10200.f + x * (1635.f + x * (150.f + x * 6.f)))))))));
}

struct Shifted {  // what the three functions share for one argument
  float y, ry, z, ln_y, d, rd;
};
__device__ __forceinline__ Shifted shift6(float x, bool want_log) {
  Shifted s;
  s.y = x + 6.0f;
  s.ry = f_rcp(s.y);
  s.z = s.ry * s.ry;
  s.ln_y = want_log ? f_log(s.y) : 0.f;
  s.d = poly_d6(x);
  s.rd = f_rcp(s.d);
  return s;
}
__device__ __forceinline__ float digamma_of(float x, const Shifted& s) {
  const float tail = s.z * (8.33333333e-2f - s.z * (8.33333333e-3f - s.z * 3.96825397e-3f));
  return s.ln_y - 0.5f * s.ry - tail - poly_n5(x) * s.rd;
}
__device__ __forceinline__ float trigamma_of(float x, const Shifted& s) {
  const float asym = s.ry + 0.5f * s.z + s.ry * s.z * (1.66666667e-1f - s.z * (3.33333333e-2f - s.z * 2.38095238e-2f));
  return asym + (poly_p10(x) * s.rd) * s.rd;
}
// lgamma(x+6) by Stirling's series; lgamma(x) = stirling - ln D(x)
__device__ __forceinline__ float stirling_of(const Shifted& s) {
  return (s.y - 0.5f) * s.ln_y - s.y + 0.918938533204672742f +
         s.ry * (8.33333333e-2f - s.z * (2.77777778e-3f - s.z * 7.93650794e-4f));
}

__device__ __forceinline__ bool fast_ok(float lo, float hi) { return lo >= kFastLo && hi <= kFastHi; }

// Entity-side quantities of KL(Beta(a,b) || .): lb = lgamma(a+b) - lgamma(a) - lgamma(b) and the
// three digammas.  One call shares the shifted arguments, logarithms and reciprocals.
static __device__ __noinline__ void beta_terms_slow(float a, float b, float& lb, float& pa, float& pb, float& ps) {
  lb = m_lgamma(a + b) - m_lgamma(a) - m_lgamma(b);
  pa = digamma(a);
  pb = digamma(b);
  ps = digamma(a + b);
}
__device__ __forceinline__ void beta_terms(float a, float b, float& lb, float& pa, float& pb, float& ps) {
  const float sum = a + b;
  if (fast_ok(fminf(a, b), sum)) {
    const Shifted sa = shift6(a, true), sb = shift6(b, true), ss = shift6(sum, true);
    pa = digamma_of(a, sa);
    pb = digamma_of(b, sb);
    ps = digamma_of(sum, ss);
    lb = (stirling_of(ss) - stirling_of(sa)) - stirling_of(sb) - f_log(ss.d * sa.rd * sb.rd);
  } else {
    beta_terms_slow(a, b, lb, pa, pb, ps);
  }
}

static __device__ __noinline__ void digamma3_slow(float a, float b, float& pa, float& pb, float& ps) {
  pa = digamma(a);
  pb = digamma(b);
  ps = digamma(a + b);
}
__device__ __forceinline__ void digamma3(float a, float b, float& pa, float& pb, float& ps) {
  const float sum = a + b;
  if (fast_ok(fminf(a, b), sum)) {
    pa = digamma_of(a, shift6(a, true));
    pb = digamma_of(b, shift6(b, true));
    ps = digamma_of(sum, shift6(sum, true));
  } else {
    digamma3_slow(a, b, pa, pb, ps);
  }
}

static __device__ __noinline__ void trigamma3_slow(float a, float b, float& ta, float& tb, float& ts) {
  ta = trigamma(a);
  tb = trigamma(b);
  ts = trigamma(a + b);
}
__device__ __forceinline__ void trigamma3(float a, float b, float& ta, float& tb, float& ts) {
  const float sum = a + b;
  if (fast_ok(fminf(a, b), sum)) {
    ta = trigamma_of(a, shift6(a, false));
    tb = trigamma_of(b, shift6(b, false));
    ts = trigamma_of(sum, shift6(sum, false));
  } else {
    trigamma3_slow(a, b, ta, tb, ts);
  }
}

}  // namespace smx
