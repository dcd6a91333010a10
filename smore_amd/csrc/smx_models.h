// Score models of the gather-fused path: logit = gamma - distance, one struct per
// model, built from the per-feature terms in smx_functors.h.
//
//   model      logit                                   reference call site
//   L1         gamma - sum |e-q|                        smore/models/vec.py:85-90
//   L2         gamma - sqrt(sum (e-q)^2)                smore/common/torchext/dist_func/l2_dist.py:59-62
//   BOX        gamma - d_out - cen * d_in               smore/models/box.py:157-164
//   ROTATE     gamma - sum sqrt(dre^2 + dim^2 + 1e-20)  smore/models/rotate.py:137-142
//   BETA_KL    gamma - sum KL(Beta(e) || Beta(q))       smore/models/beta.py:303-308
//   COMPLEX    gamma + sum (e_re q_re + e_im q_im)      smore/models/complex.py:140-148 (a similarity; gamma = 0 there)
//   DISTMULT   gamma + sum e q                          smore/models/distmult.py (distmult_sim; gamma = 0 there)
//
// A model exposes
//   fwd(e1,e2,q,acc0,acc1)      add one feature's term(s) to the lane's accumulators
//   fold(acc0,acc1,p)           the lane's single value to be summed over the wavefront
//   score(sum,p)                logit from that sum
//   coef(g,score,p,c0,c1)       d logit-loss / d accumulator, from the upstream
//                               gradient g of the logit and the saved logit
//   bwd_e / bwd_q               add one feature's gradient w.r.t. entity / query
// Optional entity prologue (BetaE): e' = clamp(e + add, lo, hi)
// (smore/common/modules.py:29-36 applied at smore/models/kg_reasoning.py:352);
// its backward passes gradient where lo <= e + add <= hi.
#pragma once
#include "../../include/smore_amd.h"
#include "smx_functors.h"

namespace smx {

enum Model : int { mL1 = 0, mL2 = 1, mBox = 2, mRotate = 3, mBetaKL = 4, mComplex = 5, mDistmult = 6, mNumModels = 7 };

__host__ __device__ constexpr int model_mul(int m) { return (m == mRotate || m == mBetaKL || m == mComplex) ? 2 : 1; }
__host__ __device__ constexpr int model_nq(int m) { return (m == mL1 || m == mL2 || m == mDistmult) ? 1 : 2; }
// models whose entity derivative can be kept as sign codes (ModelOps<M>::bwd_q_coded / bwd_e_coded)
__host__ __device__ constexpr bool model_coded(int m) { return m == mBox || m == mL1; }

struct ScoreParams {
  float gamma;
  float cen;      // weight of the inside distance (BOX only)
  int reg_on;     // entity prologue on/off
  float reg_add, reg_lo, reg_hi;
  int norm_on;    // COMPLEX, DISTMULT: unit-length halves / rows (the kernels' REG instantiation stands for it there)
};

inline ScoreParams to_params(const smx_score_params* c) {
  return ScoreParams{c->gamma, c->cen, c->reg_on, c->reg_add, c->reg_lo, c->reg_hi, c->norm_on ? 1 : 0};
}
// the entity-side options a model does not have: nullptr, or what to tell the caller
inline const char* params_refused(int model, const smx_score_params* c);

__device__ __forceinline__ float reg_apply(float e, const ScoreParams& p) {
  if (!p.reg_on) return e;
  const float v = e + p.reg_add;
  return fminf(fmaxf(v, p.reg_lo), p.reg_hi);
}
__device__ __forceinline__ float reg_mask(float e_raw, float g, const ScoreParams& p) {
  if (!p.reg_on) return g;
  const float v = e_raw + p.reg_add;
  return (v >= p.reg_lo && v <= p.reg_hi) ? g : 0.0f;
}

inline const char* params_refused(int model, const smx_score_params* c) {
  if (c->reg_on && model != mBetaKL) return "the entity clamp prologue exists for the beta_kl model only";
  if (c->norm_on && model != mComplex && model != mDistmult)
    return "unit-length rows exist for the complex and distmult models only";
  return nullptr;
}

// per-feature query registers kept by a lane for the whole tile
struct QPair {
  float a, b;
};

template <int M> struct ModelOps;

// Hook applied once to a lane's accumulated query gradient before it leaves the registers
// (identity unless a model defers part of its derivative, as BOX does).
template <int M>
__device__ __forceinline__ void finish_query_grad(const typename ModelOps<M>::Q& q, float& g1, float& g2,
                                                  const ScoreParams& p);

// ---- sign codes -----------------------------------------------------------------------------
// Models whose entity derivative is a choice among a few values (L1: +-c0; box: +-c0, +-c1) can keep
// that choice as two bits per feature -- lower bit "outside" (box only), upper bit "negative" -- one
// byte per float4 column; the features of a column are pushed in ascending order, so the last one
// sits in bits 0-1 and feature x of VEC at position VEC-1-x.
// push2: code = 4 * code + 2 * (lane's bit of hi) + (lane's bit of lo): two v_addc with the masks as
// carry-in.  The s_nop covers the wait states a VALU read of an SGPR needs after a VALU compare
// wrote it (the assembler does not look into inline asm).
__device__ __forceinline__ unsigned push2(unsigned code, unsigned long long hi, unsigned long long lo) {
  unsigned long long carry;
  asm("s_nop 1\n\t"
      "v_addc_co_u32_e64 %0, %1, %0, %0, %2\n\t"
      "v_addc_co_u32_e64 %0, %1, %0, %0, %3"
      : "+v"(code), "=&s"(carry)
      : "s"(hi), "s"(lo));
  return code;
}
// the "negative" bit of position x as a sign-bit mask
__device__ __forceinline__ unsigned code_sign(unsigned code, int x) { return (code << (30 - 2 * x)) & 0x80000000u; }

template <> struct ModelOps<mL1> {
  using Q = QPair;
  static __device__ __forceinline__ Q prep(float q1, float) { return {q1, 0.f}; }
  static __device__ __forceinline__ void fwd(float e1, float, const Q& q, float& a0, float&) {
    a0 += Term<kL1, float>::fwd(e1, 0.f, q.a, 0.f);
  }
  static __device__ __forceinline__ float fold(float a0, float, const ScoreParams&) { return a0; }
  static __device__ __forceinline__ float score(float folded, const ScoreParams& p) { return p.gamma - folded; }
  static __device__ __forceinline__ void coef(float g, float, const ScoreParams&, float& c0, float& c1) {
    c0 = -g;
    c1 = 0.f;
  }
  static __device__ __forceinline__ void bwd_e(float c0, float, float e1, float, const Q& q, float& ge1, float&) {
    float s1 = 0, s2 = 0, s3 = 0;
    Term<kL1, float>::bwd(c0, e1, 0.f, q.a, 0.f, ge1, s1, s2, s3);
  }
  static __device__ __forceinline__ void bwd_q(float c0, float, float e1, float, const Q& q, float& gq1, float&) {
    float s1 = 0, s2 = 0, s3 = 0;
    Term<kL1, float>::bwd(c0, e1, 0.f, q.a, 0.f, s1, s2, gq1, s3);
  }
  // sign codes: the derivative is c0 where e - q > 0 and -c0 elsewhere (sign(0) = -1, dist_kernel.h:141)
  static __device__ __forceinline__ float neg_threshold(const Q&) { return 0.f; }
  static __device__ __forceinline__ void fwd_coded(float e1, const Q& q, float, float& a0, float&, unsigned& code) {
    const float d = e1 - q.a;
    a0 += fabsf(d);
    code = push2(code, __ballot(!(d > 0.f)), 0ull);
  }
  static __device__ __forceinline__ void bwd_q_coded(float c0, float, float e1, const Q& q, float, float& gq1, float&,
                                                     unsigned& code) {
    const float d = e1 - q.a;
    const bool pos = d > 0.f;
    gq1 -= pos ? c0 : -c0;
    code = push2(code, __ballot(!pos), 0ull);
  }
  static __device__ __forceinline__ void bwd_q_from_code(float c0, float, unsigned code, int x, float& gq1, float&) {
    gq1 -= __uint_as_float(__float_as_uint(c0) ^ code_sign(code, x));
  }
  static __device__ __forceinline__ void bwd_e_coded(float c0, float, unsigned code, int x, float& ge) {
    ge += __uint_as_float(__float_as_uint(c0) ^ code_sign(code, x));
  }
};

template <> struct ModelOps<mL2> {
  using Q = QPair;
  static __device__ __forceinline__ Q prep(float q1, float) { return {q1, 0.f}; }
  static __device__ __forceinline__ void fwd(float e1, float, const Q& q, float& a0, float&) {
    a0 += Term<kL2, float>::fwd(e1, 0.f, q.a, 0.f);
  }
  static __device__ __forceinline__ float fold(float a0, float, const ScoreParams&) { return a0; }
  // (the root as the hardware instruction, one ulp: the correctly rounded sqrtf is a third of this model's forward)
  static __device__ __forceinline__ float score(float folded, const ScoreParams& p) {
    return p.gamma - __builtin_amdgcn_sqrtf(folded);
  }
  // d(gamma - sqrt(d2)) / d d2 = -1 / (2 sqrt(d2)): the kernels multiply this upstream part by the
  // pair's own 1 / (2 sqrt(d2)), see l2_pair_coef.  At d2 == 0 the coefficient is infinite, as autograd
  // of torch.sqrt makes it in the reference.
  static __device__ __forceinline__ void coef(float g, float, const ScoreParams&, float& c0, float& c1) {
    c0 = -g;
    c1 = 0.f;
  }
  static __device__ __forceinline__ void bwd_e(float c0, float, float e1, float, const Q& q, float& ge1, float&) {
    float s1 = 0, s2 = 0, s3 = 0;
    Term<kL2, float>::bwd(c0, e1, 0.f, q.a, 0.f, ge1, s1, s2, s3);
  }
  static __device__ __forceinline__ void bwd_q(float c0, float, float e1, float, const Q& q, float& gq1, float&) {
    float s1 = 0, s2 = 0, s3 = 0;
    Term<kL2, float>::bwd(c0, e1, 0.f, q.a, 0.f, s1, s2, gq1, s3);
  }
};

// Query2box: acc0 = outside distance, acc1 = inside distance; one row read serves both.
//
// With d = e - c, a = |d|, the terms of smore/common/torchext/dist_kernel.h:58-105 are
//   out = relu(a - o) = a - min(a, o)      (bit-identical: a - o when a > o, else a - a = 0)
//   in  = |min(a, o)|
// and their derivatives, with "outside" := (a - o >= 0), c0 / c1 the coefficients on out / in:
//   outside:  d/de = s_out c0,  d/dc = -s_out c0,  d/do = -c0 + sgn(o) c1   s_out = (d > 0 ? 1 : -1), sgn(o) = (o > 0 ? 1 : -1)
//   inside :  d/de = s_in  c1,  d/dc = -s_in  c1,  d/do = 0                 s_in  = (d >= 0 ? 1 : -1)
// (inside means a < o, so min(a,o) = a, the outer sign of the reference is -1 exactly when a == 0,
// where its inner sign is -1 too: the product is +1 there and sgn(d) elsewhere, i.e. s_in.)
// The offset gradient of a whole query is therefore (sgn(o) cen - 1) * sum over outside pairs of
// c0, so the loop only accumulates that sum and the factor is applied once at the end.
template <> struct ModelOps<mBox> {
  using Q = QPair;  // a = center, b = offset
  static __device__ __forceinline__ Q prep(float q1, float q2) { return {q1, q2}; }
  // min(|d|, o) as the one hardware instruction (fminf semantics for NaN); the compiler's own fminf
  // re-canonicalises the loop-invariant offset for every row
  static __device__ __forceinline__ float min_abs(float d, float o) {
    float mn;
    asm("v_min_f32_e64 %0, |%1|, %2" : "=v"(mn) : "v"(d), "v"(o));
    return mn;
  }
  static __device__ __forceinline__ void fwd(float e1, float, const Q& q, float& a0, float& a1) {
    const float d = e1 - q.a;
    const float a = fabsf(d);
    const float mn = min_abs(d, q.b);
    a0 += a - mn;
    a1 += fabsf(mn);
  }
  static __device__ __forceinline__ float fold(float a0, float a1, const ScoreParams& p) { return a0 + p.cen * a1; }
  static __device__ __forceinline__ float score(float folded, const ScoreParams& p) { return p.gamma - folded; }
  static __device__ __forceinline__ void coef(float g, float, const ScoreParams& p, float& c0, float& c1) {
    c0 = -g;
    c1 = -p.cen * g;
  }
  // gradient of the entity feature; the center's is its negative:
  //   outside (|d| >= o) ? (d > 0 ? c0 : -c0) : (d >= 0 ? c1 : -c1)
  // The two sign rules differ at d == 0 only, and there "outside" means o <= 0: so the sign is  d > t  with
  // t = 0 where o <= 0 and the largest negative float where o > 0 (d > t is then d >= 0), which is -o clamped
  // to [t_min, 0] -- one v_med3 instead of a second compare and a select.
  static __device__ __forceinline__ float de(float c0, float c1, float e1, const Q& q, bool& outside) {
    const float d = e1 - q.a;
    outside = fabsf(d) >= q.b;
    const float mag = outside ? c0 : c1;
    const float t = __builtin_amdgcn_fmed3f(-q.b, __uint_as_float(0x80000001u), 0.f);
    return d > t ? mag : -mag;
  }
  static __device__ __forceinline__ void bwd_e(float c0, float c1, float e1, float, const Q& q, float& ge1, float&) {
    bool outside;
    ge1 += de(c0, c1, e1, q, outside);
  }
  // gc accumulates the center gradient; go accumulates sum(c0 over outside pairs), see finish_q
  static __device__ __forceinline__ void bwd_q(float c0, float c1, float e1, float, const Q& q, float& gc, float& go) {
    bool outside;
    gc -= de(c0, c1, e1, q, outside);
    go += outside ? c0 : 0.f;
  }
  // The same for a kernel that keeps the query in registers: the sign decision of de() is one compare against
  // the feature's neg_threshold (below), which such a kernel computes once per query instead of two compares
  // and a select per pair.  Same decisions for finite operands, same +-c terms, same bits.
  static __device__ __forceinline__ void bwd_q_thr(float c0, float c1, float e1, const Q& q, float neg_thr, float& gc,
                                                   float& go) {
    const float d = e1 - q.a;
    const bool outside = fabsf(d) >= q.b;
    const float mag = outside ? c0 : c1;
    gc -= d < neg_thr ? -mag : mag;
    go += outside ? c0 : 0.f;
  }
  static __device__ __forceinline__ void finish_q(const Q& q, float&, float& go, const ScoreParams& p) {
    go *= (q.b > 0.f ? p.cen : -p.cen) - 1.0f;
  }

  // ---- sign codes ----
  // The derivative of a pair's distance w.r.t. one entity feature is +-c0 or +-c1: two bits say which.
  // The kernels that make these decisions anyway (forward, or the query-gradient kernel) can leave
  // them behind, one byte per four features; the entity pass then sums  +-c  straight from the codes
  // and needs neither the query rows nor the comparisons -- same decisions, same bits.
  // As bwd_q_thr, and pushes this feature's two bits onto `code`.
  static __device__ __forceinline__ void bwd_q_coded(float c0, float c1, float e1, const Q& q, float neg_thr, float& gc,
                                                     float& go, unsigned& code) {
    const float d = e1 - q.a;
    const bool outside = fabsf(d) >= q.b, neg = d < neg_thr;
    const float mag = outside ? c0 : c1;
    gc -= neg ? -mag : mag;
    go += outside ? c0 : 0.f;
    code = push2(code, __ballot(neg), __ballot(outside));
  }
  // As fwd, and pushes this feature's two bits onto `code`: the forward pass
  // can leave the codes too, and then the whole backward works from them without the entity rows.
  // neg_thr (per query feature, loop-invariant): the "negative" decision  outside ? d <= 0 : d < 0  is
  // d < neg_thr with neg_thr = 0 where the offset is positive (d == 0 is then inside the box) and the
  // smallest positive float where it is not (d == 0 is then outside, and d < that means d <= 0): one
  // compare instead of two compares and three mask operations.
  static __device__ __forceinline__ float neg_threshold(const Q& q) { return q.b > 0.f ? 0.f : __uint_as_float(1u); }
  static __device__ __forceinline__ void fwd_coded(float e1, const Q& q, float neg_thr, float& a0, float& a1,
                                                   unsigned& code) {
    const float d = e1 - q.a;
    const float a = fabsf(d);
    const float mn = min_abs(d, q.b);
    a0 += a - mn;
    a1 += fabsf(mn);
    code = push2(code, __ballot(d < neg_thr), __ballot(a >= q.b));
  }
  // (t ? c0 : c1) with its sign flipped when the feature's "negative" bit is set: two three-input bit
  // operations (v_bitop3_b32; table index = src0 << 2 | src1 << 1 | src2).
  static __device__ __forceinline__ float signed_pick(float c0, float c1, unsigned t, unsigned code, int x) {
    const unsigned w = __builtin_amdgcn_bitop3_b32(t, __float_as_uint(c0), __float_as_uint(c1), 0xCA);  // t ? c0 : c1
    const unsigned top = code << (30 - 2 * x);                                    // "negative" bit in bit 31
    return __uint_as_float(__builtin_amdgcn_bitop3_b32(w, top, 0x80000000u, 0x78));  // w ^ (top & sign bit)
  }
  // Query side from a code byte: gc -= derivative of the feature at position x, go += c0 where the pair is outside.
  static __device__ __forceinline__ void bwd_q_from_code(float c0, float c1, unsigned code, int x, float& gc,
                                                         float& go) {
    const unsigned t = (unsigned)__builtin_amdgcn_sbfe((int)code, 2 * x, 1);  // 0 or ~0
    gc -= signed_pick(c0, c1, t, code, x);
    go += __uint_as_float(__float_as_uint(c0) & t);
  }
  // ge += derivative of the feature at position x of the lane's code byte
  static __device__ __forceinline__ void bwd_e_coded(float c0, float c1, unsigned code, int x, float& ge) {
    const unsigned t = (unsigned)__builtin_amdgcn_sbfe((int)code, 2 * x, 1);  // 0 or ~0
    ge += signed_pick(c0, c1, t, code, x);
  }
};

template <> struct ModelOps<mRotate> {
  using Q = QPair;  // a = re, b = im
  static __device__ __forceinline__ Q prep(float q1, float q2) { return {q1, q2}; }
  static __device__ __forceinline__ void fwd(float e1, float e2, const Q& q, float& a0, float&) {
    a0 += Term<kRotate, float>::fwd(e1, e2, q.a, q.b);
  }
  static __device__ __forceinline__ float fold(float a0, float, const ScoreParams&) { return a0; }
  static __device__ __forceinline__ float score(float folded, const ScoreParams& p) { return p.gamma - folded; }
  static __device__ __forceinline__ void coef(float g, float, const ScoreParams&, float& c0, float& c1) {
    c0 = -g;
    c1 = 0.f;
  }
  static __device__ __forceinline__ void bwd_e(float c0, float, float e1, float e2, const Q& q, float& ge1, float& ge2) {
    float s1 = 0, s2 = 0;
    Term<kRotate, float>::bwd(c0, e1, e2, q.a, q.b, ge1, ge2, s1, s2);
  }
  static __device__ __forceinline__ void bwd_q(float c0, float, float e1, float e2, const Q& q, float& g1, float& g2) {
    float s1 = 0, s2 = 0;
    Term<kRotate, float>::bwd(c0, e1, e2, q.a, q.b, s1, s2, g1, g2);
  }
};

// BetaE: KL(Beta(ea,eb) || Beta(qa,qb)) of smore/common/torchext/dist_kernel.h:207-266, regrouped into an
// entity part and a query part so that everything that depends on one side only is evaluated once:
//   KL = [lgG(qa)+lgG(qb)-lgG(sq)] + [lgG(se)-lgG(ea)-lgG(eb)] + (ea-qa)psi(ea) + (eb-qb)psi(eb) + (sq-se)psi(se)
//   dKL/dqa = [psi(qa) - psi(sq)] - psi(ea) + psi(se)                       (same with b)
//   dKL/dea = (ea-qa) psi'(ea) + (sq-se) psi'(se)                            (same with b)
// The bracketed query terms are per (query, feature) constants held in the lane's query registers.
// For the entity gradient the trigammas depend on the entity only, and (ea-qa) + (eb-qb) = se - sq,
// so a segment accumulates S1 = sum c (ea-qa), S2 = sum c (eb-qb) and applies
//   g_a = psi'(ea) S1 - psi'(se) (S1+S2),  g_b = psi'(eb) S2 - psi'(se) (S1+S2)
// once when the segment is finished.
struct QBeta {
  float a, b;  // alpha, beta of the query
  float k;     // forward: lgG(qa)+lgG(qb)-lgG(sq); query backward: psi(qa)-psi(sq)
  float l;     // query backward: psi(qb)-psi(sq)
};

template <> struct ModelOps<mBetaKL> {
  using Q = QBeta;
  static __device__ __forceinline__ Q prep(float q1, float q2) { return {q1, q2, 0.f, 0.f}; }
  static __device__ __forceinline__ Q prep_fwd(float q1, float q2) {
    float lb, pa, pb, ps;
    beta_terms(q1, q2, lb, pa, pb, ps);
    return {q1, q2, -lb, 0.f};
  }
  static __device__ __forceinline__ Q prep_bwd_q(float q1, float q2) {
    float pa, pb, ps;
    digamma3(q1, q2, pa, pb, ps);
    return {q1, q2, pa - ps, pb - ps};
  }
  static __device__ __forceinline__ void fwd(float ea, float eb, const Q& q, float& a0, float&) {
    float lb, pa, pb, ps;
    beta_terms(ea, eb, lb, pa, pb, ps);
    a0 += (q.k + lb) + (ea - q.a) * pa + (eb - q.b) * pb + ((q.a + q.b) - (ea + eb)) * ps;
  }
  static __device__ __forceinline__ float fold(float a0, float, const ScoreParams&) { return a0; }
  static __device__ __forceinline__ float score(float folded, const ScoreParams& p) { return p.gamma - folded; }
  static __device__ __forceinline__ void coef(float g, float, const ScoreParams&, float& c0, float& c1) {
    c0 = -g;
    c1 = 0.f;
  }
  // accumulates S1, S2 (see above); finish_e turns them into the gradient
  static __device__ __forceinline__ void bwd_e(float c0, float, float e1, float e2, const Q& q, float& s1, float& s2) {
    s1 += c0 * (e1 - q.a);
    s2 += c0 * (e2 - q.b);
  }
  static __device__ __forceinline__ void finish_e(float e1, float e2, float& g1, float& g2) {
    float ta, tb, ts;
    trigamma3(e1, e2, ta, tb, ts);
    const float common = ts * (g1 + g2);
    g1 = ta * g1 - common;
    g2 = tb * g2 - common;
  }
  static __device__ __forceinline__ void bwd_q(float c0, float, float e1, float e2, const Q& q, float& g1, float& g2) {
    float pa, pb, ps;
    digamma3(e1, e2, pa, pb, ps);
    g1 += c0 * (q.k - pa + ps);
    g2 += c0 * (q.l - pb + ps);
  }
};

// ComplEx and DistMult score by similarity, not distance (dist_kernel.h:187-204, 324-349): the logit grows
// with the inner product, so the upstream coefficient keeps its sign.
template <> struct ModelOps<mComplex> {
  using Q = QPair;  // a = re, b = im
  static __device__ __forceinline__ Q prep(float q1, float q2) { return {q1, q2}; }
  static __device__ __forceinline__ void fwd(float e1, float e2, const Q& q, float& a0, float&) {
    a0 += Term<kComplex, float>::fwd(e1, e2, q.a, q.b);
  }
  static __device__ __forceinline__ float fold(float a0, float, const ScoreParams&) { return a0; }
  static __device__ __forceinline__ float score(float folded, const ScoreParams& p) { return p.gamma + folded; }
  static __device__ __forceinline__ void coef(float g, float, const ScoreParams&, float& c0, float& c1) {
    c0 = g;
    c1 = 0.f;
  }
  static __device__ __forceinline__ void bwd_e(float c0, float, float e1, float e2, const Q& q, float& ge1, float& ge2) {
    float s1 = 0, s2 = 0;
    Term<kComplex, float>::bwd(c0, e1, e2, q.a, q.b, ge1, ge2, s1, s2);
  }
  static __device__ __forceinline__ void bwd_q(float c0, float, float e1, float e2, const Q& q, float& g1, float& g2) {
    float s1 = 0, s2 = 0;
    Term<kComplex, float>::bwd(c0, e1, e2, q.a, q.b, s1, s2, g1, g2);
  }
};

// ComplEx with unit-length halves (complex.py:142-146 when the model's mode names 'norm', complex.py:87-89;
// embed_norm = F.normalize(p = 2, dim = -1), modules.py:38-40):
//   logit = gamma + (re . q_re) / max(|re|, eps) + (im . q_im) / max(|im|, eps),   eps = 1e-12
//   d logit / d q_re = re / max(|re|, eps)
//   d logit / d re   = (q_re - re_n (re_n . q_re)) / |re|   with re_n = re / |re|    (q_re / eps below eps)
// The scaling belongs to the entity, not to the pair: summed over an entity's pairs the gradient is the plain ComplEx
// gradient G = sum c q pushed through the scaling once, g_re = (G_re - re_n (re_n . G_re)) / |re|.  The entity
// kernels therefore accumulate G as they do for plain ComplEx, and the function that finishes a row applies the
// projection.  In the kernels the REG instantiation of the ComplEx model stands for this form.
// DistMult's 'norm' mode (distmult.py:85-87,129-130) is the same with the whole row as its only half:
//   logit = gamma + (e . q) / max(|e|, eps).
constexpr float kNormEps = 1e-12f;
__host__ __device__ constexpr bool model_norm(int m, bool reg) { return (m == mComplex || m == mDistmult) && reg; }
__device__ __forceinline__ float inv_norm(float sumsq) { return 1.f / fmaxf(__builtin_sqrtf(sumsq), kNormEps); }

template <> struct ModelOps<mDistmult> {
  using Q = QPair;
  static __device__ __forceinline__ Q prep(float q1, float) { return {q1, 0.f}; }
  static __device__ __forceinline__ void fwd(float e1, float, const Q& q, float& a0, float&) {
    a0 += Term<kDistmult, float>::fwd(e1, 0.f, q.a, 0.f);
  }
  static __device__ __forceinline__ float fold(float a0, float, const ScoreParams&) { return a0; }
  static __device__ __forceinline__ float score(float folded, const ScoreParams& p) { return p.gamma + folded; }
  static __device__ __forceinline__ void coef(float g, float, const ScoreParams&, float& c0, float& c1) {
    c0 = g;
    c1 = 0.f;
  }
  static __device__ __forceinline__ void bwd_e(float c0, float, float e1, float, const Q& q, float& ge1, float&) {
    float s1 = 0, s2 = 0, s3 = 0;
    Term<kDistmult, float>::bwd(c0, e1, 0.f, q.a, 0.f, ge1, s1, s2, s3);
  }
  static __device__ __forceinline__ void bwd_q(float c0, float, float e1, float, const Q& q, float& gq1, float&) {
    float s1 = 0, s2 = 0, s3 = 0;
    Term<kDistmult, float>::bwd(c0, e1, 0.f, q.a, 0.f, s1, s2, gq1, s3);
  }
};

// Query registers for the forward / the query-backward kernel (models without side constants use prep).
template <int M>
__device__ __forceinline__ typename ModelOps<M>::Q prep_forward(float q1, float q2) {
  if constexpr (M == mBetaKL) return ModelOps<M>::prep_fwd(q1, q2);
  else return ModelOps<M>::prep(q1, q2);
}
template <int M>
__device__ __forceinline__ typename ModelOps<M>::Q prep_backward_query(float q1, float q2) {
  if constexpr (M == mBetaKL) return ModelOps<M>::prep_bwd_q(q1, q2);
  else return ModelOps<M>::prep(q1, q2);
}

// Hook applied once per finished entity row to the summed accumulators (identity unless a model
// defers part of its derivative, as BETA_KL does).  e1 / e2 are the (regularised) entity values.
template <int M>
__device__ __forceinline__ void finish_entity_grad(float e1, float e2, float& g1, float& g2) {
  if constexpr (M == mBetaKL) ModelOps<mBetaKL>::finish_e(e1, e2, g1, g2);
}

template <int M>
__device__ __forceinline__ void finish_query_grad(const typename ModelOps<M>::Q& q, float& g1, float& g2,
                                                  const ScoreParams& p) {
  if constexpr (M == mBox) ModelOps<mBox>::finish_q(q, g1, g2, p);
}

}  // namespace smx
