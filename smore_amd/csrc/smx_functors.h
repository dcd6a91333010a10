// Per-feature distance terms and their derivatives.
//
// One struct per operator kind; each mirrors one functor of the operator set
// being replaced (smore/common/torchext/dist_kernel.h, lines cited per kind).
// Entity rows of the "two halves" kinds are laid out [first | second], each
// half `dim` long (dist_kernel.h:37-55), so a term sees e1 = row[d] and
// e2 = row[d + dim]; q1 / q2 are the two query tensors at feature d.
//
// Subgradient conventions at ties are those of the replaced kernels, not of
// autograd: sign(0) = -1, box_out passes gradient when |e-c|-o == 0, box_in
// sends |e-c| == o to the offset branch.
#pragma once
#include "smx_math.h"

namespace smx {

enum Kind : int {
  kL1 = 0,
  kL2 = 1,  // squared; the caller takes the root
  kBoxOut = 2,
  kBoxIn = 3,
  kRotate = 4,
  kBetaKL = 5,
  kComplex = 6,
  kDistmult = 7,
  kBetaL2 = 8,
  kBetaFisher = 9,
  kNumKinds = 10
};

__host__ __device__ constexpr int kind_mul(int k) {
  return (k == kRotate || k == kBetaKL || k == kComplex || k == kBetaL2 || k == kBetaFisher) ? 2 : 1;
}
__host__ __device__ constexpr int kind_nq(int k) {
  return (k == kL1 || k == kL2 || k == kDistmult) ? 1 : 2;
}

template <int K, typename T> struct Term;

// dist_kernel.h:129-155
template <typename T> struct Term<kL1, T> {
  static __device__ __forceinline__ T fwd(T e1, T, T q1, T) { return m_abs(e1 - q1); }
  static __device__ __forceinline__ void bwd(T g, T e1, T, T q1, T, T& ge1, T&, T& gq1, T&) {
    const T s = (e1 - q1 > 0) ? g : -g;
    ge1 += s;
    gq1 -= s;
  }
};

// dist_kernel.h:158-184
template <typename T> struct Term<kL2, T> {
  static __device__ __forceinline__ T fwd(T e1, T, T q1, T) {
    const T a = e1 - q1;
    return a * a;
  }
  static __device__ __forceinline__ void bwd(T g, T e1, T, T q1, T, T& ge1, T&, T& gq1, T&) {
    const T t = g * (e1 - q1) * (T)2;
    ge1 += t;
    gq1 -= t;
  }
};

// dist_kernel.h:58-79
template <typename T> struct Term<kBoxOut, T> {
  static __device__ __forceinline__ T fwd(T e, T, T c, T o) {
    const T r = m_abs(e - c) - o;
    return r > 0 ? r : (T)0;
  }
  static __device__ __forceinline__ void bwd(T g, T e, T, T c, T o, T& ge, T&, T& gc, T& go) {
    if (m_abs(e - c) - o >= 0) {
      go -= g;
      const T s = (e - c > 0) ? g : -g;
      ge += s;
      gc -= s;
    }
  }
};

// dist_kernel.h:82-105
template <typename T> struct Term<kBoxIn, T> {
  static __device__ __forceinline__ T fwd(T e, T, T c, T o) { return m_abs(m_min(m_abs(e - c), o)); }
  static __device__ __forceinline__ void bwd(T g, T e, T, T c, T o, T& ge, T&, T& gc, T& go) {
    const T da = m_abs(e - c);
    const T og = (m_min(da, o) > 0) ? g : -g;
    if (da < o) {
      const T s = (e - c > 0) ? og : -og;
      ge += s;
      gc -= s;
    } else {
      go += og;
    }
  }
};

// dist_kernel.h:108-126; the 1e-20 inside the root is cuda_math_ext.h:21,100-118
// fp32: the root and the reciprocal root as the hardware's own instructions (v_sqrt_f32, v_rsq_f32: one ulp), as the
// CUDA kernels use sqrtf / rsqrtf of the same argument; the argument is at least 1e-20, far above the subnormals.
// (The correctly rounded sqrtf and the IEEE division of the C library forms cost some twenty instructions per
// feature: 25 of the forward's and 35 of the backward's per complex feature were those.)
template <typename T> struct Term<kRotate, T> {
  static __device__ __forceinline__ T fwd(T e1, T e2, T q1, T q2) {
    const T a = e1 - q1, b = e2 - q2;
    if constexpr (sizeof(T) == sizeof(float)) return __builtin_amdgcn_sqrtf(a * a + b * b + 1e-20f);
    else return m_sqrt(a * a + b * b + (T)1e-20);
  }
  static __device__ __forceinline__ void bwd(T g, T e1, T e2, T q1, T q2, T& ge1, T& ge2, T& gq1, T& gq2) {
    const T a = e1 - q1, b = e2 - q2;
    T r;
    if constexpr (sizeof(T) == sizeof(float)) r = g * __builtin_amdgcn_rsqf(a * a + b * b + 1e-20f);
    else r = g / m_sqrt(a * a + b * b + (T)1e-20);
    ge1 += a * r;
    ge2 += b * r;
    gq1 -= a * r;
    gq2 -= b * r;
  }
};

// dist_kernel.h:187-204
template <typename T> struct Term<kComplex, T> {
  static __device__ __forceinline__ T fwd(T e1, T e2, T q1, T q2) { return e1 * q1 + e2 * q2; }
  static __device__ __forceinline__ void bwd(T g, T e1, T e2, T q1, T q2, T& ge1, T& ge2, T& gq1, T& gq2) {
    ge1 += q1 * g;
    ge2 += q2 * g;
    gq1 += e1 * g;
    gq2 += e2 * g;
  }
};

// dist_kernel.h:324-349
template <typename T> struct Term<kDistmult, T> {
  static __device__ __forceinline__ T fwd(T e1, T, T q1, T) { return e1 * q1; }
  static __device__ __forceinline__ void bwd(T g, T e1, T, T q1, T, T& ge1, T&, T& gq1, T&) {
    ge1 += q1 * g;
    gq1 += e1 * g;
  }
};

// dist_kernel.h:207-266.  KL(Beta(e1,e2) || Beta(q1,q2)).  The backward is the
// closed form of the term-by-term code there (its +g*psi / -g*psi pairs cancel):
//   d/de1 = (e1-q1) psi'(e1) + (Sq-Se) psi'(Se)      d/dq1 = psi(q1) - psi(e1) + psi(Se) - psi(Sq)
template <typename T> struct Term<kBetaKL, T> {
  static __device__ __forceinline__ T fwd(T ea, T eb, T qa, T qb) {
    const T se = ea + eb, sq = qa + qb;
    const T t1 = m_lgamma(qa) + m_lgamma(qb) + m_lgamma(se);
    const T t2 = m_lgamma(ea) + m_lgamma(eb) + m_lgamma(sq);
    return t1 - t2 + (ea - qa) * digamma(ea) + (eb - qb) * digamma(eb) + (sq - se) * digamma(se);
  }
  static __device__ __forceinline__ void bwd(T g, T ea, T eb, T qa, T qb, T& gea, T& geb, T& gqa, T& gqb) {
    const T se = ea + eb, sq = qa + qb;
    const T common_e = (sq - se) * trigamma(se);
    gea += g * ((ea - qa) * trigamma(ea) + common_e);
    geb += g * ((eb - qb) * trigamma(eb) + common_e);
    const T common_q = digamma(se) - digamma(sq);
    gqa += g * (digamma(qa) - digamma(ea) + common_q);
    gqb += g * (digamma(qb) - digamma(eb) + common_q);
  }
};

// fp32: the same closed forms on the shared fast evaluations of smx_math.h (one call per Beta
// distribution gives its three digammas or trigammas and its log-Beta term without a data-dependent loop).
template <> struct Term<kBetaKL, float> {
  static __device__ __forceinline__ float fwd(float ea, float eb, float qa, float qb) {
    float lbe, pa, pb, ps, lbq, ua, ub, us;
    beta_terms(ea, eb, lbe, pa, pb, ps);   // lbe = lgamma(se) - lgamma(ea) - lgamma(eb)
    beta_terms(qa, qb, lbq, ua, ub, us);   // only lbq is used
    return (lbe - lbq) + (ea - qa) * pa + (eb - qb) * pb + ((qa + qb) - (ea + eb)) * ps;
  }
  static __device__ __forceinline__ void bwd(float g, float ea, float eb, float qa, float qb, float& gea, float& geb,
                                             float& gqa, float& gqb) {
    const float se = ea + eb, sq = qa + qb;
    float ta, tb, ts, pa, pb, ps, ua, ub, us;
    trigamma3(ea, eb, ta, tb, ts);
    digamma3(ea, eb, pa, pb, ps);
    digamma3(qa, qb, ua, ub, us);
    const float common_e = (sq - se) * ts;
    gea += g * ((ea - qa) * ta + common_e);
    geb += g * ((eb - qb) * tb + common_e);
    const float common_q = ps - us;
    gqa += g * (ua - pa + common_q);
    gqb += g * (ub - pb + common_q);
  }
};

// dist_kernel.h:269-287
template <typename T> struct Term<kBetaL2, T> {
  static __device__ __forceinline__ T fwd(T e1, T e2, T q1, T q2) {
    const T a = e1 - q1, b = e2 - q2;
    return (T)0.5 * (a * a + b * b);
  }
  static __device__ __forceinline__ void bwd(T g, T e1, T e2, T q1, T q2, T& ge1, T& ge2, T& gq1, T& gq2) {
    const T a = g * (e1 - q1), b = g * (e2 - q2);
    ge1 += a;
    ge2 += b;
    gq1 -= a;
    gq2 -= b;
  }
};

// dist_kernel.h:290-321.  The trigamma weights are constants for the backward.
template <typename T> struct Term<kBetaFisher, T> {
  static __device__ __forceinline__ T fwd(T ea, T eb, T qa, T qb) {
    const T pa = trigamma(ea), pb = trigamma(eb), nab = -trigamma(ea + eb);
    const T da = ea - qa, db = eb - qb;
    return (T)0.5 * (da * da * (pa + nab) + 2 * nab * da * db + db * db * (pb + nab));
  }
  static __device__ __forceinline__ void bwd(T g, T ea, T eb, T qa, T qb, T& gea, T& geb, T& gqa, T& gqb) {
    const T pa = trigamma(ea), pb = trigamma(eb), nab = -trigamma(ea + eb);
    const T da = ea - qa, db = eb - qb;
    const T m = nab * (da + db);
    const T gl = g * (pa * da + m), gr = g * (pb * db + m);
    gea += gl;
    geb += gr;
    gqa -= gl;
    gqb -= gr;
  }
};

template <> struct Term<kBetaFisher, float> {
  static __device__ __forceinline__ float fwd(float ea, float eb, float qa, float qb) {
    float pa, pb, ps;
    trigamma3(ea, eb, pa, pb, ps);
    const float nab = -ps, da = ea - qa, db = eb - qb;
    return 0.5f * (da * da * (pa + nab) + 2 * nab * da * db + db * db * (pb + nab));
  }
  static __device__ __forceinline__ void bwd(float g, float ea, float eb, float qa, float qb, float& gea, float& geb,
                                             float& gqa, float& gqb) {
    float pa, pb, ps;
    trigamma3(ea, eb, pa, pb, ps);
    const float nab = -ps, da = ea - qa, db = eb - qb;
    const float m = nab * (da + db);
    const float gl = g * (pa * da + m), gr = g * (pb * db + m);
    gea += gl;
    geb += gr;
    gqa -= gl;
    gqb -= gr;
  }
};

}  // namespace smx
