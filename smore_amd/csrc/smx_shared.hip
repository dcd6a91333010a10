// Entity-side backward for negatives shared by the whole batch: host side (see smx_shared_impl.h).
#include "smx_shared_impl.h"

namespace smx {

extern template int shared_entity_dispatch<mL1>(hipStream_t, const SharedArgs&, int, int);
extern template int shared_entity_dispatch<mL2>(hipStream_t, const SharedArgs&, int, int);
extern template int shared_entity_dispatch<mBox>(hipStream_t, const SharedArgs&, int, int);
extern template int shared_entity_dispatch<mRotate>(hipStream_t, const SharedArgs&, int, int);
extern template int shared_entity_dispatch<mBetaKL>(hipStream_t, const SharedArgs&, int, int);
extern template int shared_entity_dispatch<mComplex>(hipStream_t, const SharedArgs&, int, int);
extern template int shared_entity_dispatch<mDistmult>(hipStream_t, const SharedArgs&, int, int);

// defined in smx_shared_gemm.hip
bool shared_gemm_fits(int model, size_t dim, const void* table, const void* q1, const void* q2, const void* workspace,
                      size_t workspace_bytes, size_t B, size_t K, bool entity, bool norm);
int shared_gemm_entity_sums(int model, hipStream_t st, const float* q1, const float* q2, const float* gscore, size_t B,
                            size_t K, size_t dim, float* workspace);

}  // namespace smx

extern "C" int smx_score_backward_entity_shared(int model, void* stream, float* table, size_t n_rows, const int64_t* ids,
                                                const float* q1, const float* q2, const float* score,
                                                const float* gscore, size_t B, size_t K, size_t dim,
                                                const smx_score_params* params, const smx_plan_view* plan,
                                                float* grad_rows, float* merged, float* m, float* v,
                                                const smx_opt_params* adam, void* workspace, size_t workspace_bytes) {
  using namespace smx;
  if (model < 0 || model >= mNumModels) return fail(SMX_ERR_KIND, "unknown score model %d", model);
  if (!table || !ids || !q1 || !score || !gscore || !params || (model_nq(model) == 2 && !q2))
    return fail(SMX_ERR_ARG, "null pointer");
  if (B == 0 || K == 0 || dim == 0 || n_rows == 0) return fail(SMX_ERR_SHAPE, "empty dimension");
  if (B > 0x7fffffffull || K > 0x7fffffffull || B * K > 0x7fffffffull)
    return fail(SMX_ERR_SHAPE, "more than 2^31-1 pairs in one call");
  if (const char* why = params_refused(model, params)) return fail(SMX_ERR_ARG, "%s", why);
  SharedArgs A{};
  if (plan) {
    if (grad_rows) return fail(SMX_ERR_ARG, "gradient rows per list position are the output of the call without a plan");
    if (!merged && !adam) return fail(SMX_ERR_ARG, "nothing to do: neither merged gradient nor an optimizer requested");
    if (!plan->order || !plan->seg_start || !plan->uniq || !plan->n_uniq) return fail(SMX_ERR_ARG, "incomplete segment plan");
    if (plan->n_pairs != K) return fail(SMX_ERR_SHAPE, "the plan must be built over the %zu shared ids, it holds %zu", K, plan->n_pairs);
    A.by_segment = 1;
    A.order = plan->order;
    A.seg_start = plan->seg_start;
    A.uniq = reinterpret_cast<const long long*>(plan->uniq);
    A.n_uniq = plan->n_uniq;
    A.merged = merged;
  } else {
    if (!grad_rows) return fail(SMX_ERR_ARG, "without a plan the call writes one gradient row per list position: grad_rows is null");
    if (merged || adam || m || v) return fail(SMX_ERR_ARG, "merged rows and the optimizer update need the segment plan of the ids");
    A.merged = grad_rows;
  }
  A.adam_on = 0;
  A.m = m;
  A.v = v;
  if (adam) {
    if (const char* msg = check_opt_params(adam, m, v)) return fail(SMX_ERR_ARG, "%s", msg);
    A.adam_on = adam->kind;
    A.squeeze = adam->squeeze ? 1 : 0;
    A.a = make_adam_consts(adam);
    A.step_dev = adam->step_consts_dev;
  } else if (m || v) {
    return fail(SMX_ERR_ARG, "optimizer state given without optimizer parameters");
  }
  const bool vec4 = dim % 4 == 0 && aligned16(table) && aligned16(q1) && (!q2 || aligned16(q2)) &&
                    (!A.merged || aligned16(A.merged)) && (!m || aligned16(m)) &&
                    (!v || (adam && adam->squeeze) || aligned16(v));
  const int vec = vec4 ? 4 : 1;
  const size_t ncol = dim / vec;
  if (ncol > 512) return fail(SMX_ERR_SHAPE, "dim %zu not supported by the fused path", dim);
  const int need = (int)((ncol + 63) / 64);
  const int nit = need <= 1 ? 1 : (need <= 2 ? 2 : (need <= 4 ? 4 : 8));
  if (vec == 1 && nit > 4) return fail(SMX_ERR_SHAPE, "rows of %zu unaligned floats are not supported by the fused path", (size_t)ncol);
  A.ids = reinterpret_cast<const long long*>(ids);
  A.q1 = q1;
  A.q2 = q2;
  A.score = score;
  A.gscore = gscore;
  A.B = (int)B;
  A.K = (int)K;
  A.n_rows = n_rows;
  A.p = to_params(params);
  A.table = table;
  A.ncol = (int)ncol;
  hipStream_t st = as_stream(stream);
  // BetaE, ComplEx, DistMult: the sums over the queries as a matrix product into the workspace, finished row by row below
  if (vec == 4 && shared_gemm_fits(model, dim, table, q1, q2, workspace, workspace_bytes, B, K, true, false)) {
    float* ws = static_cast<float*>(workspace);
    if (int rc = shared_gemm_entity_sums(model, st, q1, q2, gscore, B, K, dim, ws)) return rc;
    A.sums_r = ws;
    A.sums_c = ws + K * (size_t)model_nq(model) * dim;
  }
  switch (model) {
    case mL1: return shared_entity_dispatch<mL1>(st, A, vec, nit);
    case mL2: return shared_entity_dispatch<mL2>(st, A, vec, nit);
    case mBox: return shared_entity_dispatch<mBox>(st, A, vec, nit);
    case mRotate: return shared_entity_dispatch<mRotate>(st, A, vec, nit);
    case mBetaKL: return shared_entity_dispatch<mBetaKL>(st, A, vec, nit);
    case mComplex: return shared_entity_dispatch<mComplex>(st, A, vec, nit);
    case mDistmult: return shared_entity_dispatch<mDistmult>(st, A, vec, nit);
  }
  return fail(SMX_ERR_KIND, "unknown score model %d", model);
}
