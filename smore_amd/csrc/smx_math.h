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

__device__ __forceinline__ float m_log(float x) { return __logf(x); }
__device__ __forceinline__ double m_log(double x) { return log(x); }
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

}  // namespace smx
