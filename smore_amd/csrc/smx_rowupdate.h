// Finishing one entity row: the pieces shared by the entity pass (smx_entity_impl.h) and by the
// query-backward kernel when it finishes one-pair segments itself (smx_score_impl.h).
//
// "Finishing" = turning the summed accumulators of a segment into the row's gradient (model hook,
// clamp mask), storing it as a merged-gradient row and/or applying the lazy Adam update of
// smore/common/embedding/embed_optimizer.py:208-252 to the w, m, v rows in place.
#pragma once
#include <cmath>

#include "../../include/smore_amd.h"
#include "smx_models.h"
#include "smx_wave.h"

namespace smx {

constexpr int kSrcRows = 100;  // source = materialised gradient rows instead of a score model

__host__ __device__ constexpr int src_mul(int s) { return s == kSrcRows ? 1 : model_mul(s); }

// Row optimizers of smore/common/embedding/embed_optimizer.py (all lazy: touched rows only).
//   Adam     :208-252   m' = b1 m + (1-b1) g, v' = b2 v + (1-b2) g2, w += -(lr/bc1) m' / (sqrt(v')/sqrt(bc2) + eps)
//   SGD      :174-178   w += -lr g
//   AdaGrad  :327-349   v' = v + g2,                w += -lr g / (sqrt(v') + eps)
//   RMSprop  :271-309   v' = a v + (1-a) g2,        w += -lr g / (sqrt(v') + eps)        (a = beta2 field)
// g2 = g*g per feature, or with `squeeze` the row mean of g*g, v then being one value per row.
enum OptKind : int { kOptNone = 0, kOptAdam = SMX_OPT_ADAM, kOptSgd = SMX_OPT_SGD, kOptAdagrad = SMX_OPT_ADAGRAD,
                     kOptRmsprop = SMX_OPT_RMSPROP };

struct AdamConsts {
  float beta1, beta2, omb1, omb2, eps, step_size, inv_sqrt_bc2;
};

inline AdamConsts make_adam_consts(const smx_opt_params* a) {
  AdamConsts c;
  const bool adam = a->kind == SMX_OPT_ADAM;
  const double bc1 = adam ? 1.0 - std::pow(a->beta1, (double)a->step) : 1.0;
  const double bc2 = adam ? 1.0 - std::pow(a->beta2, (double)a->step) : 1.0;
  c.beta1 = (float)a->beta1;
  c.beta2 = (float)a->beta2;
  c.omb1 = (float)(1.0 - a->beta1);
  c.omb2 = (float)(1.0 - a->beta2);
  c.eps = (float)a->eps;
  c.step_size = (float)(-a->lr / bc1);
  c.inv_sqrt_bc2 = (float)(1.0 / std::sqrt(bc2));
  return c;
}

// The two constants that change from step to step (learning rate and Adam's bias corrections), as a
// caller may keep them in device memory: { -lr / (1 - beta1^step), 1 / sqrt(1 - beta2^step) }.
inline void step_consts(const smx_opt_params* a, float out[2]) {
  const AdamConsts c = make_adam_consts(a);
  out[0] = c.step_size;
  out[1] = c.inv_sqrt_bc2;
}

// Square root and reciprocal of the update's denominator as the single hardware instructions (1 ulp
// each) instead of the correctly rounded sequences (about ten instructions each): the step they scale
// is added to a weight hundreds of times its size, so the weight changes by far less than one ulp of
// difference, and the row update is a fifth shorter.  m and v, which carry over to the next step, are
// computed exactly as before.
__device__ __forceinline__ float hw_sqrt(float x) { return __builtin_amdgcn_sqrtf(x); }
__device__ __forceinline__ float hw_rcp(float x) { return __builtin_amdgcn_rcpf(x); }

// L2 only.  score = gamma - sqrt(d2), so d score / d d2 = -1 / (2 sqrt(d2)).  The reference divides by the
// square root autograd saved (l2_dist.py:59,62); recovering it as gamma - score would add half an ulp of
// gamma to the distance, a relative error of 5e-7 / distance.  The backward kernels hold the pair's entity
// row and query in registers anyway, so they sum d2 again, in the forward's order, and multiply by its reciprocal root.
// c_raw: the upstream part of the coefficient (-gscore).  e(it, v), q(it, v): the lane's features.
template <int VEC, int NIT, class GetE, class GetQ>
__device__ __forceinline__ float l2_pair_coef(float c_raw, int ncol, int lane, GetE&& e, GetQ&& q) {
  float mine = 0.f;
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    float a0 = 0.f;
#pragma unroll
    for (int v = 0; v < VEC; ++v) a0 += Term<kL2, float>::fwd(e(it, v), 0.f, q(it, v), 0.f);
    mine += lane + 64 * it < ncol ? a0 : 0.f;
  }
  const float d2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(wave_sum_last_f32(mine)), 63));
  return c_raw * (0.5f * __builtin_amdgcn_rsqf(d2));  // (one ulp; infinite at d2 == 0 like the division)
}

// ComplEx with unit-length halves, query backward: the pair's upstream coefficient over the two lengths of its row.
template <int VEC, int NIT, int MUL, class GetE1, class GetE2>
__device__ __forceinline__ float2 norm_pair_coef(float c_raw, int ncol, int lane, GetE1&& e1, GetE2&& e2) {
  float s1 = 0.f, s2 = 0.f;
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    float a = 0.f, b = 0.f;
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      a = __builtin_fmaf(e1(it, v), e1(it, v), a);
      if constexpr (MUL == 2) b = __builtin_fmaf(e2(it, v), e2(it, v), b);
    }
    const bool in = lane + 64 * it < ncol;
    s1 += in ? a : 0.f;
    s2 += in ? b : 0.f;
  }
  const float c1 = c_raw * inv_norm(wave_sum_f32(s1));
  if constexpr (MUL == 1) return make_float2(c1, 0.f);  // (DistMult: the row is its only half)
  return make_float2(c1, c_raw * inv_norm(wave_sum_f32(s2)));
}

// ... entity side: the summed plain gradient g of one half row w pushed through w / max(|w|, eps)
template <int VEC, int NIT, class GetW>
__device__ __forceinline__ void norm_project(float (&g)[NIT][VEC], int ncol, int lane, GetW&& w) {
  float sq = 0.f, dot = 0.f;
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    float a = 0.f, b = 0.f;
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      a = __builtin_fmaf(w(it, v), w(it, v), a);
      b = __builtin_fmaf(w(it, v), g[it][v], b);
    }
    const bool in = lane + 64 * it < ncol;
    sq += in ? a : 0.f;
    dot += in ? b : 0.f;
  }
  sq = wave_sum_f32(sq);
  dot = wave_sum_f32(dot);
  const float len = __builtin_sqrtf(sq);
  const bool live = len > kNormEps;  // below eps the scaling is the constant 1 / eps
  const float inv = live ? 1.f / len : 1.f / kNormEps;
  const float k = live ? dot * inv * inv : 0.f;
#pragma unroll
  for (int it = 0; it < NIT; ++it)
#pragma unroll
    for (int v = 0; v < VEC; ++v) g[it][v] = (g[it][v] - w(it, v) * k) * inv;
}

// 0 when the parameters are usable, else a message for the caller
inline const char* check_opt_params(const smx_opt_params* a, const void* m, const void* v) {
  if (a->kind < SMX_OPT_ADAM || a->kind > SMX_OPT_RMSPROP) return "unknown optimizer kind";
  if (a->kind == SMX_OPT_ADAM && a->step < 1) return "Adam step counter starts at 1";
  if (a->kind == SMX_OPT_ADAM && !m) return "Adam needs the first-moment table m";
  if (a->kind != SMX_OPT_SGD && !v) return "this optimizer needs the state table v";
  return nullptr;
}

// Where finished rows go.
struct RowSink {
  float* table;   // entity table: read for the model sources, updated when an optimizer is on
  float* m;       // Adam first moment [N, row]
  float* v;       // second moment / squared-gradient state: [N, row], or [N] with squeeze
  float* merged;  // [U, row_len] or null
  int adam_on;    // OptKind; 0 = no optimizer (name kept from the Adam-only version)
  int squeeze;
  AdamConsts a;
  const float* step_dev;  // null, or device memory holding { step_size, inv_sqrt_bc2 } that replace a's
  ScoreParams p;
  int ncol;       // columns per half row (model sources) or per row (gradient rows)
};

template <int VEC> struct Pack2 {
  float v[VEC];
};

// STREAM marks data that crosses the chip once per step (optimizer state, rows of one-off partial
// sums, the updated rows written back): loaded and stored with the non-temporal hint, it does not push
// the rows that are reused (queries, popular entities) out of the L2.
typedef float vec4f __attribute__((ext_vector_type(4)));

template <int VEC, bool STREAM = false>
__device__ __forceinline__ Pack2<VEC> ld(const float* __restrict__ base, int col) {
  Pack2<VEC> r;
  if constexpr (VEC == 4) {
    const vec4f* p = reinterpret_cast<const vec4f*>(base) + col;
    const vec4f t = STREAM ? __builtin_nontemporal_load(p) : *p;
    r.v[0] = t.x;
    r.v[1] = t.y;
    r.v[2] = t.z;
    r.v[3] = t.w;
  } else {
    r.v[0] = STREAM ? __builtin_nontemporal_load(base + col) : base[col];
  }
  return r;
}

template <int VEC, bool STREAM = false>
__device__ __forceinline__ void st(float* __restrict__ base, int col, const float (&x)[VEC]) {
  if constexpr (VEC == 4) {
    vec4f t;
    t.x = x[0];
    t.y = x[1];
    t.z = x[2];
    t.w = x[3];
    vec4f* p = reinterpret_cast<vec4f*>(base) + col;
    if (STREAM) __builtin_nontemporal_store(t, p);
    else *p = t;
  } else {
    if (STREAM) __builtin_nontemporal_store(x[0], base + col);
    else base[col] = x[0];
  }
}

// The lane's columns of one table row (both halves for the two-half models).
template <int MUL, int VEC, int NIT> struct RowRegs {
  Pack2<VEC> h[MUL][NIT];
};

template <int MUL, int VEC, int NIT, bool STREAM = false>
__device__ __forceinline__ void load_row(RowRegs<MUL, VEC, NIT>& r, const float* __restrict__ base, int half, int ncol,
                                         int lane) {
#pragma unroll
  for (int h = 0; h < MUL; ++h)
#pragma unroll
    for (int it = 0; it < NIT; ++it) r.h[h][it] = ld<VEC, STREAM>(base + h * half, min(lane + 64 * it, ncol - 1));
}

// finish_row's default for `extra`: nothing to add
struct NoExtraRows {
  template <class G> __device__ __forceinline__ void operator()(G&, G&) const {}
};

// Finishes one entity row: clamp mask, merged-gradient store, Adam.  g1/g2 are the lane's columns of
// the summed gradient of the first / second half row; w, m0, v0 the row's current weights and moments
// (w is always valid for the model sources -- it is the entity row the gradient was computed from).
// ADAM_STATIC: the caller knows at compile time that Adam is on (its m0 / v0 are loaded); otherwise the
// run-time flag A.adam_on decides.  extra(g1, g2): adds what reaches the row from outside the score model
// (gradient rows of the step's plain lookups) once the model's own gradient is complete, clamp mask included.
template <int SRC, int VEC, int NIT, bool REG, bool ADAM_STATIC = false, class Extra = NoExtraRows>
__device__ __forceinline__ void finish_row(const RowSink& A, int lane, unsigned row_id, int seg,
                                           float (&g1)[NIT][VEC], float (&g2)[NIT][VEC],
                                           const RowRegs<src_mul(SRC), VEC, NIT>& w,
                                           const RowRegs<src_mul(SRC), VEC, NIT>& m0,
                                           const RowRegs<src_mul(SRC), VEC, NIT>& v0, Extra&& extra = Extra()) {
  constexpr int MUL = src_mul(SRC);
  const int half = A.ncol * VEC;
  const size_t row_len = (size_t)half * MUL;
  if constexpr (SRC != kSrcRows) {
#pragma unroll
    for (int it = 0; it < NIT; ++it)
#pragma unroll
      for (int x = 0; x < VEC; ++x) {
        const float x1 = REG ? reg_apply(w.h[0][it].v[x], A.p) : w.h[0][it].v[x];
        const float x2 = MUL == 2 ? (REG ? reg_apply(w.h[MUL - 1][it].v[x], A.p) : w.h[MUL - 1][it].v[x]) : 0.f;
        finish_entity_grad<SRC>(x1, x2, g1[it][x], g2[it][x]);
      }
    if constexpr (model_norm(SRC, REG)) {
      norm_project<VEC, NIT>(g1, A.ncol, lane, [&](int it, int x) { return w.h[0][it].v[x]; });
      if constexpr (MUL == 2) norm_project<VEC, NIT>(g2, A.ncol, lane, [&](int it, int x) { return w.h[MUL - 1][it].v[x]; });
    }
  }
  if (REG) {
#pragma unroll
    for (int it = 0; it < NIT; ++it)
#pragma unroll
      for (int x = 0; x < VEC; ++x) {
        g1[it][x] = reg_mask(w.h[0][it].v[x], g1[it][x], A.p);
        if (MUL == 2) g2[it][x] = reg_mask(w.h[MUL - 1][it].v[x], g2[it][x], A.p);
      }
  }
  extra(g1, g2);
  if (A.merged) {
    float* out = A.merged + (size_t)seg * row_len;
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      const int c = lane + 64 * it;
      if (c < A.ncol) {
        st<VEC, true>(out, c, g1[it]);
        if (MUL == 2) st<VEC, true>(out + half, c, g2[it]);
      }
    }
  }
  if (ADAM_STATIC || A.adam_on) {
    const int kind = A.adam_on;
    // per-step constants: from the launch arguments, or read now from the caller's device buffer (so that a
    // captured launch follows the learning-rate schedule and the step counter between replays)
    const float step_size = A.step_dev ? A.step_dev[0] : A.a.step_size;
    const float inv_sqrt_bc2 = A.step_dev ? A.step_dev[1] : A.a.inv_sqrt_bc2;
    float* pw = A.table + (size_t)row_id * row_len;
    float* pm = A.m + (size_t)row_id * row_len;
    float* pv = A.v + (size_t)row_id * row_len;
    float g2_row = 0.f, v_row = 0.f;
    if (A.squeeze && kind != kOptSgd) {  // one second-moment value per row, fed by the row mean of g*g
      float part = 0.f;
#pragma unroll
      for (int it = 0; it < NIT; ++it)
        if (lane + 64 * it < A.ncol) {
#pragma unroll
          for (int x = 0; x < VEC; ++x) {
            part = __builtin_fmaf(g1[it][x], g1[it][x], part);
            if (MUL == 2) part = __builtin_fmaf(g2[it][x], g2[it][x], part);
          }
        }
      g2_row = wave_sum_f32(part) / (float)row_len;
      v_row = A.v[row_id];
    }
    float v_new_row = 0.f;
#pragma unroll
    for (int h = 0; h < MUL; ++h) {
#pragma unroll
      for (int it = 0; it < NIT; ++it) {
        const int c = lane + 64 * it;
        if (c < A.ncol) {
          float wn[VEC], mn[VEC], vn[VEC];
#pragma unroll
          for (int x = 0; x < VEC; ++x) {
            const float g = h == 0 ? g1[it][x] : g2[it][x];
            const float gg = A.squeeze ? g2_row : g * g;
            const float v_old = A.squeeze ? v_row : v0.h[h][it].v[x];
            // Every multiply-add is written as the fused operation it is meant to be: left to the
            // compiler's contraction, the kernels that share this function round a*b + c*d differently
            // from one another, and the same row would get different bits depending on which one finishes it.
            if (kind == kOptAdam) {
              mn[x] = __builtin_fmaf(m0.h[h][it].v[x], A.a.beta1, g * A.a.omb1);
              vn[x] = __builtin_fmaf(v_old, A.a.beta2, gg * A.a.omb2);
              const float denom = __builtin_fmaf(hw_sqrt(vn[x]), inv_sqrt_bc2, A.a.eps);
              wn[x] = __builtin_fmaf(step_size * mn[x], hw_rcp(denom), w.h[h][it].v[x]);
            } else if (kind == kOptSgd) {
              mn[x] = vn[x] = 0.f;
              wn[x] = __builtin_fmaf(step_size, g, w.h[h][it].v[x]);
            } else {
              mn[x] = 0.f;
              vn[x] = kind == kOptAdagrad ? v_old + gg : __builtin_fmaf(v_old, A.a.beta2, gg * A.a.omb2);
              wn[x] = __builtin_fmaf(step_size * g, hw_rcp(hw_sqrt(vn[x]) + A.a.eps), w.h[h][it].v[x]);
            }
            v_new_row = vn[x];
          }
          st<VEC, true>(pw + h * half, c, wn);
          if (kind == kOptAdam) st<VEC, true>(pm + h * half, c, mn);
          if (kind != kOptSgd && !A.squeeze) st<VEC, true>(pv + h * half, c, vn);
        }
      }
    }
    if (A.squeeze && kind != kOptSgd && lane == 0) A.v[row_id] = v_new_row;
  }
}

template <int MUL, int VEC, int NIT> struct RowState {
  RowRegs<MUL, VEC, NIT> e, m, v;
};

template <int SRC, int VEC, int NIT>
__device__ __forceinline__ void request_state(const RowSink& A, int lane, unsigned row_id,
                                              RowState<src_mul(SRC), VEC, NIT>& s) {
  constexpr int MUL = src_mul(SRC);
  const int half = A.ncol * VEC;
  const size_t off = (size_t)row_id * half * MUL;
  if (SRC != kSrcRows || A.adam_on) load_row<MUL, VEC, NIT, true>(s.e, A.table + off, half, A.ncol, lane);
  if (A.adam_on == kOptAdam) load_row<MUL, VEC, NIT, true>(s.m, A.m + off, half, A.ncol, lane);
  if (A.adam_on && A.adam_on != kOptSgd && !A.squeeze) load_row<MUL, VEC, NIT, true>(s.v, A.v + off, half, A.ncol, lane);
}

}  // namespace smx
