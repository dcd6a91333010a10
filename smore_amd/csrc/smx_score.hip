// Gather-fused scoring, forward and query-side backward (fp32).
//
// Replaces, in one pass each, the sequence the reference runs per training
// step for the negative samples (smore/models/kg_reasoning.py:301-307,349-355):
//   rows = table[idx]                      smore/common/embedding/embed_rw.py:74-75
//   [optional clamp(rows + 1, .05, 1e9)]   smore/common/modules.py:29-36
//   d = dist(rows, query)                  smore/common/torchext/common_kernel.h:33-56
//   logit = gamma - d                      custom_cal_logit of smore/models/*.py
// and, backward, the query-gradient kernel common_kernel.h:92-123.  The
// [B,K,D] gathered tensor is never materialised: a wavefront reads each entity
// row straight from the table with 16-byte loads (one float4 column per lane).
//
// Work split.  forward: workgroup = (query b, tile of negatives); the query
// row(s) are staged once in LDS, every lane then keeps the features it owns in
// registers for the whole tile; each of the four wavefronts streams its
// quarter of the tile's rows, two batches of rows in flight at a time.  backward: one workgroup per
// query walks all K negatives, wavefront partial sums are combined through LDS
// in wavefront order, so the gradient has a fixed summation order.
#include "smx_common.h"
#include "smx_models.h"
#include "smx_wave.h"

namespace smx {

template <int VEC> struct Pack {
  float v[VEC];
};

template <int VEC>
__device__ __forceinline__ Pack<VEC> load_pack(const float* __restrict__ base, int col) {
  Pack<VEC> r;
  if constexpr (VEC == 4) {
    const float4 t = reinterpret_cast<const float4*>(base)[col];
    r.v[0] = t.x;
    r.v[1] = t.y;
    r.v[2] = t.z;
    r.v[3] = t.w;
  } else {
    r.v[0] = base[col];
  }
  return r;
}

// Loads the features a lane owns of the staged query into registers.
template <int M, int VEC, int NIT, bool FWD>
__device__ __forceinline__ void load_query_regs(const float* lds, int dim, int ncol, int lane,
                                                typename ModelOps<M>::Q (&q)[NIT][VEC]) {
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    const int c = lane + 64 * it;
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      const int cc = min(c, ncol - 1);  // lanes past the row end hold a copy of the last column
      const float a = lds[cc * VEC + v];
      const float b = model_nq(M) == 2 ? lds[dim + cc * VEC + v] : 0.f;
      q[it][v] = FWD ? prep_forward<M>(a, b) : prep_backward_query<M>(a, b);
    }
  }
}

template <int M>
__device__ __forceinline__ void stage_query(float* lds, const float* __restrict__ q1, const float* __restrict__ q2,
                                            size_t b, int dim) {
  for (int d = threadIdx.x; d < dim; d += blockDim.x) {
    lds[d] = q1[b * dim + d];
    if (model_nq(M) == 2) lds[dim + d] = q2[b * dim + d];
  }
  __syncthreads();
}

// ---- streaming the rows of up to 64 pairs through a wavefront -----------------------------------
// The lanes first fetch, in one coalesced load, the ids of the pairs the wavefront is about to
// process (pair j of the batch lives in lane j) and turn them into row offsets.  The row loop then
// needs no memory access to find a row: the offset comes out of lane j with two v_readlane, so the
// only loads in the loop are the rows themselves.  Rows are requested RIF at a time into two
// register sets used in turn: while set A is consumed, set B is already on its way.  All loads are
// unconditional (indices are clamped) so that they issue as one batch and stay in flight together.

struct PairBatch {
  unsigned off_lo, off_hi;  // this lane's pair: offset of its entity row in floats
};

__device__ __forceinline__ PairBatch load_pair_batch(const long long* __restrict__ idx, size_t first_pair, int cnt,
                                                     int lane, size_t row_len, unsigned long long n_rows, int& bad) {
  const size_t pair = first_pair + min(lane, cnt - 1);
  long long row = idx ? idx[pair] : (long long)pair;
  if ((unsigned long long)row >= n_rows) {  // id outside the table: remember it, read row 0 instead
    bad = 1;
    row = 0;
  }
  const unsigned long long off = (unsigned long long)row * row_len;
  return {(unsigned)off, (unsigned)(off >> 32)};
}

__device__ __forceinline__ const float* batch_row(const float* __restrict__ table, const PairBatch& pb, int j) {
  const unsigned lo = (unsigned)__builtin_amdgcn_readlane((int)pb.off_lo, j);
  const unsigned hi = (unsigned)__builtin_amdgcn_readlane((int)pb.off_hi, j);
  return table + (((unsigned long long)hi << 32) | lo);
}

template <int MUL, int VEC, int NIT, int RIF> struct RowSet {
  Pack<VEC> e1[RIF][NIT];
  Pack<VEC> e2[RIF][NIT];
};

// Requests rows j0 .. j0+RIF-1 of the batch (clamped to cnt-1).
template <int MUL, int VEC, int NIT, int RIF>
__device__ __forceinline__ void request_rows(RowSet<MUL, VEC, NIT, RIF>& rs, const float* __restrict__ table,
                                             const PairBatch& pb, int j0, int cnt, int dim, int ncol, int lane) {
#pragma unroll
  for (int r = 0; r < RIF; ++r) {
    const float* pe = batch_row(table, pb, min(j0 + r, cnt - 1));
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      const int c = min(lane + 64 * it, ncol - 1);
      rs.e1[r][it] = load_pack<VEC>(pe, c);
      if (MUL == 2) rs.e2[r][it] = load_pack<VEC>(pe + dim, c);
    }
  }
}

// Streams the cnt (<= 64) rows of a batch through `consume(j, e1, e2)`, j ascending.
template <int MUL, int VEC, int NIT, int RIF, class Consume>
__device__ __forceinline__ void stream_batch(const float* __restrict__ table, const PairBatch& pb, int cnt, int dim,
                                             int ncol, int lane, Consume&& consume) {
  RowSet<MUL, VEC, NIT, RIF> a, b;
  const int last = ((cnt - 1) / RIF) * RIF;  // first row of the last group
  request_rows<MUL, VEC, NIT, RIF>(a, table, pb, 0, cnt, dim, ncol, lane);
  for (int j0 = 0; j0 < cnt; j0 += 2 * RIF) {
    request_rows<MUL, VEC, NIT, RIF>(b, table, pb, min(j0 + RIF, last), cnt, dim, ncol, lane);
#pragma unroll
    for (int r = 0; r < RIF; ++r)
      if (j0 + r < cnt) consume(j0 + r, a.e1[r], a.e2[r]);
    request_rows<MUL, VEC, NIT, RIF>(a, table, pb, min(j0 + 2 * RIF, last), cnt, dim, ncol, lane);
#pragma unroll
    for (int r = 0; r < RIF; ++r)
      if (j0 + RIF + r < cnt) consume(j0 + RIF + r, b.e1[r], b.e2[r]);
  }
}

template <int M, int VEC, int NIT, int RIF, bool REG>
__global__ __launch_bounds__(256) void score_forward_kernel(const float* __restrict__ table,
                                                            const long long* __restrict__ idx,
                                                            const float* __restrict__ q1, const float* __restrict__ q2,
                                                            float* __restrict__ score, int K, int ncol, int tiles,
                                                            int tile_k, unsigned long long n_rows, ScoreParams p,
                                                            int* err) {
  constexpr int MUL = model_mul(M);
  extern __shared__ float lds[];
  const int b = blockIdx.x / tiles;
  const int tile = blockIdx.x - b * tiles;
  const int lane = threadIdx.x & 63;
  const int wave = uniform(threadIdx.x >> 6);
  const int dim = ncol * VEC;
  const size_t row_len = (size_t)dim * MUL;

  // this wavefront's share of the tile: per_wave (<= 64) consecutive negatives
  const int per_wave = tile_k / 4;
  const int kw0 = tile * tile_k + wave * per_wave;
  const int cnt = min(per_wave, K - kw0);
  int bad = 0;
  PairBatch pb{0u, 0u};
  if (cnt > 0) pb = load_pair_batch(idx, (size_t)b * K + kw0, cnt, lane, row_len, n_rows, bad);

  stage_query<M>(lds, q1, q2, b, dim);
  typename ModelOps<M>::Q q[NIT][VEC];
  load_query_regs<M, VEC, NIT, true>(lds, dim, ncol, lane, q);
  if (cnt <= 0) return;

  float* out = score + (size_t)b * K + kw0;
  stream_batch<MUL, VEC, NIT, RIF>(table, pb, cnt, dim, ncol, lane,
                                   [&](int j, const Pack<VEC>(&e1)[NIT], const Pack<VEC>(&e2)[NIT]) {
    float a0 = 0.f, a1 = 0.f;
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      if (lane + 64 * it < ncol) {
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
          const float x1 = REG ? reg_apply(e1[it].v[v], p) : e1[it].v[v];
          const float x2 = MUL == 2 ? (REG ? reg_apply(e2[it].v[v], p) : e2[it].v[v]) : 0.f;
          ModelOps<M>::fwd(x1, x2, q[it][v], a0, a1);
        }
      }
    }
    // the logit is linear in the accumulators: fold them per lane, reduce once
    const float folded = wave_sum_f32(ModelOps<M>::fold(a0, a1, p));
    if (lane == 0) out[j] = ModelOps<M>::score(folded, p);
  });
  if (__ballot(bad != 0) != 0ull && err && lane == 0) *err = 1;
}

template <int M, int VEC, int NIT, int RIF, int NW, bool REG>
__global__ __launch_bounds__(NW * 64) void score_backward_query_kernel(
    const float* __restrict__ table, const long long* __restrict__ idx, const float* __restrict__ q1,
    const float* __restrict__ q2, const float* __restrict__ score, const float* __restrict__ gscore,
    float* __restrict__ gq1, float* __restrict__ gq2, int K, int ncol, unsigned long long n_rows, ScoreParams p) {
  constexpr int MUL = model_mul(M);
  constexpr int NQ = model_nq(M);
  extern __shared__ float lds[];
  const int b = blockIdx.x;
  const int lane = threadIdx.x & 63;
  const int wave = uniform(threadIdx.x >> 6);
  const int dim = ncol * VEC;
  const size_t row_len = (size_t)dim * MUL;

  stage_query<M>(lds, q1, q2, b, dim);
  typename ModelOps<M>::Q q[NIT][VEC];
  load_query_regs<M, VEC, NIT, false>(lds, dim, ncol, lane, q);

  float g1[NIT][VEC], g2[NIT][VEC];
#pragma unroll
  for (int it = 0; it < NIT; ++it)
#pragma unroll
    for (int v = 0; v < VEC; ++v) g1[it][v] = g2[it][v] = 0.f;

  // this wavefront's share of the query's negatives: a contiguous range, walked in batches of 64
  const int per_wave = (K + NW - 1) / NW;
  const int kw0 = wave * per_wave;
  const int kw1 = min(K, kw0 + per_wave);
  int bad = 0;
  for (int kb = kw0; kb < kw1; kb += 64) {
    const int cnt = min(64, kw1 - kb);
    const size_t first = (size_t)b * K + kb;
    const PairBatch pb = load_pair_batch(idx, first, cnt, lane, row_len, n_rows, bad);
    const size_t mine = first + min(lane, cnt - 1);
    float my_c0, my_c1;
    ModelOps<M>::coef(gscore[mine], score[mine], p, my_c0, my_c1);
    stream_batch<MUL, VEC, NIT, RIF>(table, pb, cnt, dim, ncol, lane,
                                     [&](int j, const Pack<VEC>(&e1)[NIT], const Pack<VEC>(&e2)[NIT]) {
      const float c0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(my_c0), j));
      const float c1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(my_c1), j));
#pragma unroll
      for (int it = 0; it < NIT; ++it) {
        if (lane + 64 * it < ncol) {
#pragma unroll
          for (int v = 0; v < VEC; ++v) {
            const float x1 = REG ? reg_apply(e1[it].v[v], p) : e1[it].v[v];
            const float x2 = MUL == 2 ? (REG ? reg_apply(e2[it].v[v], p) : e2[it].v[v]) : 0.f;
            ModelOps<M>::bwd_q(c0, c1, x1, x2, q[it][v], g1[it][v], g2[it][v]);
          }
        }
      }
    });
  }

#pragma unroll
  for (int it = 0; it < NIT; ++it)
#pragma unroll
    for (int v = 0; v < VEC; ++v) finish_query_grad<M>(q[it][v], g1[it][v], g2[it][v], p);

  // wavefront partials -> LDS -> fixed-order sum over wavefronts
  float* part = lds + NQ * dim;  // [NW][NQ][dim]
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    const int c = lane + 64 * it;
    if (c < ncol) {
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        part[(wave * NQ + 0) * dim + c * VEC + v] = g1[it][v];
        if (NQ == 2) part[(wave * NQ + 1) * dim + c * VEC + v] = g2[it][v];
      }
    }
  }
  __syncthreads();
  for (int d = threadIdx.x; d < dim; d += NW * 64) {
    float s1 = 0.f, s2 = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      s1 += part[(w * NQ + 0) * dim + d];
      if (NQ == 2) s2 += part[(w * NQ + 1) * dim + d];
    }
    gq1[(size_t)b * dim + d] = s1;
    if (NQ == 2) gq2[(size_t)b * dim + d] = s2;
  }
}

// ---- host dispatch ---------------------------------------------------------------------------

struct ScoreShape {
  int vec, nit, ncol;
};

// Picks the column width: float4 columns when rows are 16-byte aligned, single floats otherwise.
static int pick_shape(size_t dim, int mul, const void* table, const void* qa, const void* qb, ScoreShape* s) {
  const bool vec4 = dim % 4 == 0 && aligned16(table) && aligned16(qa) && (!qb || aligned16(qb));
  (void)mul;
  s->vec = vec4 ? 4 : 1;
  const size_t ncol = dim / s->vec;
  if (ncol > 512) return fail(SMX_ERR_SHAPE, "dim %zu not supported by the fused path (at most %d)", dim, 512 * s->vec);
  s->ncol = (int)ncol;
  const int need = (int)((ncol + 63) / 64);
  s->nit = need <= 1 ? 1 : (need <= 2 ? 2 : (need <= 4 ? 4 : 8));
  return SMX_OK;
}

static ScoreParams to_params(const smx_score_params* p) {
  ScoreParams r;
  r.gamma = p->gamma;
  r.cen = p->cen;
  r.reg_on = p->reg_on;
  r.reg_add = p->reg_add;
  r.reg_lo = p->reg_lo;
  r.reg_hi = p->reg_hi;
  return r;
}

// rows requested per batch; two batches are in flight at a time
constexpr int rows_in_flight(int nit, int mul) {
  const int r = 4 / (nit * mul);
  return r < 1 ? 1 : r;
}

template <int M, int VEC, int NIT, bool REG>
static int launch_forward_reg(hipStream_t st, const float* table, const int64_t* idx, const float* q1, const float* q2,
                          float* score, size_t B, size_t K, int ncol, size_t n_rows, const ScoreParams& p, int* err) {
  constexpr int RIF = rows_in_flight(NIT, model_mul(M));
  int tile_k = 256;  // 64 negatives per wavefront; smaller tiles when the grid would not fill the chip
  while (tile_k > 4 * RIF && (B * ((K + tile_k - 1) / tile_k) < 8192 || (size_t)tile_k / 2 >= K)) tile_k /= 2;
  const int tiles = (int)((K + tile_k - 1) / tile_k);
  const size_t lds = (size_t)model_nq(M) * ncol * VEC * sizeof(float);
  hipLaunchKernelGGL((score_forward_kernel<M, VEC, NIT, RIF, REG>), dim3((unsigned)(B * tiles)), dim3(256), lds, st, table,
                     reinterpret_cast<const long long*>(idx), q1, q2, score, (int)K, ncol, tiles, tile_k,
                     (unsigned long long)n_rows, p, err);
  return check_launch("score forward");
}

template <int M, int VEC, int NIT>
static int launch_forward(hipStream_t st, const float* table, const int64_t* idx, const float* q1, const float* q2,
                          float* score, size_t B, size_t K, int ncol, size_t n_rows, const ScoreParams& p, int* err) {
  if constexpr (M == mBetaKL) {
    if (p.reg_on) return launch_forward_reg<M, VEC, NIT, true>(st, table, idx, q1, q2, score, B, K, ncol, n_rows, p, err);
  }
  return launch_forward_reg<M, VEC, NIT, false>(st, table, idx, q1, q2, score, B, K, ncol, n_rows, p, err);
}

template <int M, int VEC, int NIT, int NW>
static int launch_backward_query(hipStream_t st, const float* table, const int64_t* idx, const float* q1,
                                 const float* q2, const float* score, const float* gscore, float* gq1, float* gq2,
                                 size_t B, size_t K, int ncol, size_t n_rows, const ScoreParams& p) {
  constexpr int RIF = rows_in_flight(NIT, model_mul(M));
  const size_t lds = (size_t)(NW + 1) * model_nq(M) * ncol * VEC * sizeof(float);
  if constexpr (M == mBetaKL) {
    if (p.reg_on) {
      hipLaunchKernelGGL((score_backward_query_kernel<M, VEC, NIT, RIF, NW, true>), dim3((unsigned)B), dim3(NW * 64),
                         lds, st, table, reinterpret_cast<const long long*>(idx), q1, q2, score, gscore, gq1, gq2,
                         (int)K, ncol, (unsigned long long)n_rows, p);
      return check_launch("score backward (query)");
    }
  }
  hipLaunchKernelGGL((score_backward_query_kernel<M, VEC, NIT, RIF, NW, false>), dim3((unsigned)B), dim3(NW * 64), lds,
                     st, table, reinterpret_cast<const long long*>(idx), q1, q2, score, gscore, gq1, gq2, (int)K, ncol,
                     (unsigned long long)n_rows, p);
  return check_launch("score backward (query)");
}

template <int M, int VEC, int NIT>
static int pick_waves_backward_query(hipStream_t st, const float* table, const int64_t* idx, const float* q1,
                                     const float* q2, const float* score, const float* gscore, float* gq1, float* gq2,
                                     size_t B, size_t K, int ncol, size_t n_rows, const ScoreParams& p) {
  const size_t per_wave = (size_t)model_nq(M) * ncol * VEC * sizeof(float);
  if (9 * per_wave <= 60 * 1024)
    return launch_backward_query<M, VEC, NIT, 8>(st, table, idx, q1, q2, score, gscore, gq1, gq2, B, K, ncol, n_rows, p);
  if (5 * per_wave <= 60 * 1024)
    return launch_backward_query<M, VEC, NIT, 4>(st, table, idx, q1, q2, score, gscore, gq1, gq2, B, K, ncol, n_rows, p);
  return launch_backward_query<M, VEC, NIT, 2>(st, table, idx, q1, q2, score, gscore, gq1, gq2, B, K, ncol, n_rows, p);
}

#define SMX_DISPATCH_NIT(M, VEC, nit, CALL) \
  switch (nit) {                            \
    case 1: return CALL(M, VEC, 1);         \
    case 2: return CALL(M, VEC, 2);         \
    case 4: return CALL(M, VEC, 4);         \
    default: return CALL(M, VEC, 8);        \
  }

#define SMX_DISPATCH_SHAPE(M, shape, CALL)       \
  if ((shape).vec == 4) {                        \
    SMX_DISPATCH_NIT(M, 4, (shape).nit, CALL)    \
  } else {                                       \
    SMX_DISPATCH_NIT(M, 1, (shape).nit, CALL)    \
  }

#define SMX_DISPATCH_MODEL(model, shape, CALL)            \
  switch (model) {                                        \
    case mL1: SMX_DISPATCH_SHAPE(mL1, shape, CALL)        \
    case mL2: SMX_DISPATCH_SHAPE(mL2, shape, CALL)        \
    case mBox: SMX_DISPATCH_SHAPE(mBox, shape, CALL)      \
    case mRotate: SMX_DISPATCH_SHAPE(mRotate, shape, CALL) \
    case mBetaKL: SMX_DISPATCH_SHAPE(mBetaKL, shape, CALL) \
  }

static int check_score_args(int model, const float* table, const float* q1, const float* q2, size_t B, size_t K,
                            size_t dim, const smx_score_params* params) {
  if (model < 0 || model >= mNumModels) return fail(SMX_ERR_KIND, "unknown score model %d", model);
  if (!table || !q1 || !params || (model_nq(model) == 2 && !q2)) return fail(SMX_ERR_ARG, "null pointer");
  if (B == 0 || K == 0 || dim == 0) return fail(SMX_ERR_SHAPE, "empty dimension");
  if (B > 0x7fffffffull || K > 0x7fffffffull || B * K > 0x7fffffffull)
    return fail(SMX_ERR_SHAPE, "more than 2^31-1 pairs in one call");
  if (params->reg_on && model != mBetaKL)
    return fail(SMX_ERR_ARG, "the entity clamp prologue exists for the beta_kl model only");
  return SMX_OK;
}

}  // namespace smx

extern "C" {

int smx_score_forward(int model, void* stream, const float* table, size_t n_rows, const int64_t* idx,
                      const float* q1, const float* q2, float* score, size_t B, size_t K, size_t dim,
                      const smx_score_params* params, int* err_flag) {
  using namespace smx;
  if (int rc = check_score_args(model, table, q1, q2, B, K, dim, params)) return rc;
  if (!score) return fail(SMX_ERR_ARG, "null score pointer");
  if (!idx) n_rows = B * K;
  ScoreShape shape;
  if (int rc = pick_shape(dim, model_mul(model), table, q1, model_nq(model) == 2 ? q2 : nullptr, &shape)) return rc;
  const ScoreParams p = to_params(params);
  hipStream_t st = as_stream(stream);
#define CALL(M, VEC, NIT) launch_forward<M, VEC, NIT>(st, table, idx, q1, q2, score, B, K, shape.ncol, n_rows, p, err_flag)
  SMX_DISPATCH_MODEL(model, shape, CALL)
#undef CALL
  return fail(SMX_ERR_KIND, "unknown score model %d", model);
}

int smx_score_backward_query(int model, void* stream, const float* table, size_t n_rows, const int64_t* idx,
                             const float* q1, const float* q2, const float* score, const float* gscore, float* gq1,
                             float* gq2, size_t B, size_t K, size_t dim, const smx_score_params* params) {
  using namespace smx;
  if (int rc = check_score_args(model, table, q1, q2, B, K, dim, params)) return rc;
  if (!score || !gscore || !gq1 || (model_nq(model) == 2 && !gq2)) return fail(SMX_ERR_ARG, "null pointer");
  if (!idx) n_rows = B * K;
  ScoreShape shape;
  if (int rc = pick_shape(dim, model_mul(model), table, q1, model_nq(model) == 2 ? q2 : nullptr, &shape)) return rc;
  const ScoreParams p = to_params(params);
  hipStream_t st = as_stream(stream);
#define CALL(M, VEC, NIT) \
  pick_waves_backward_query<M, VEC, NIT>(st, table, idx, q1, q2, score, gscore, gq1, gq2, B, K, shape.ncol, n_rows, p)
  SMX_DISPATCH_MODEL(model, shape, CALL)
#undef CALL
  return fail(SMX_ERR_KIND, "unknown score model %d", model);
}

}  // extern "C"
