// Host side of the all-entity ranking (see smx_rank_impl.h).
#include "smx_rank_impl.h"

namespace smx {

extern template int rank_dispatch<mL1>(hipStream_t, const RankArgs&, int, int, int);
extern template int rank_dispatch<mL2>(hipStream_t, const RankArgs&, int, int, int);
extern template int rank_dispatch<mBox>(hipStream_t, const RankArgs&, int, int, int);
extern template int rank_dispatch<mRotate>(hipStream_t, const RankArgs&, int, int, int);
extern template int rank_dispatch<mBetaKL>(hipStream_t, const RankArgs&, int, int, int);
extern template int rank_dispatch<mComplex>(hipStream_t, const RankArgs&, int, int, int);
extern template int rank_dispatch<mDistmult>(hipStream_t, const RankArgs&, int, int, int);

constexpr size_t kRankMaxCandidates = 4096;  // per query: their keys live in LDS
constexpr size_t kRankMaxAnswers = 2048;  // per query; bins and keys of a pass live in LDS (per query of the pass 2049 x 4 + 2048 x 8 bytes)

static size_t rank_ws_bytes(size_t B, size_t A) { return (B * (A + 1) * sizeof(unsigned) + 255) & ~(size_t)255; }

static int rank_common(RankArgs* R, int* vec, int* nit, int model, const float* table, size_t n_rows, const float* q1,
                       const float* q2, size_t B, size_t U, size_t dim, const smx_score_params* params,
                       const int64_t* ans_id, const int32_t* ans_count, size_t A) {
  if (model < 0 || model >= mNumModels) return fail(SMX_ERR_KIND, "unknown score model %d", model);
  if (!table || !q1 || !params || !ans_id || !ans_count || (model_nq(model) == 2 && !q2))
    return fail(SMX_ERR_ARG, "null pointer");
  if (B == 0 || dim == 0 || n_rows == 0 || A == 0) return fail(SMX_ERR_SHAPE, "empty dimension");
  if (U == 0 || U > (size_t)kRankQueries) return fail(SMX_ERR_SHAPE, "1 to %d union branches", kRankQueries);
  if (B * U > 0x7fffffffull) return fail(SMX_ERR_SHAPE, "too many query rows");
  if (n_rows > 0xfffffff8ull) return fail(SMX_ERR_SHAPE, "entity count %zu needs ids wider than 32 bits", n_rows);
  if (A > kRankMaxAnswers) return fail(SMX_ERR_SHAPE, "at most %zu answers per query", kRankMaxAnswers);
  if (B > 0x7fffffffull / (A + 1)) return fail(SMX_ERR_SHAPE, "too many queries");
  if (const char* why = params_refused(model, params)) return fail(SMX_ERR_ARG, "%s", why);
  const bool vec4 = dim % 4 == 0 && aligned16(table) && aligned16(q1) && (model_nq(model) == 1 || aligned16(q2));
  *vec = vec4 ? 4 : 1;
  const size_t ncol = dim / *vec;
  const int need = (int)((ncol + 63) / 64);
  *nit = need <= 1 ? 1 : (need <= 2 ? 2 : (need <= 4 ? 4 : 8));
  if (ncol > 512 || (*vec == 1 && *nit > 4))
    return fail(SMX_ERR_SHAPE, "dim %zu not supported (at most 2048 aligned or 256 unaligned floats)", dim);
  *R = RankArgs{};
  R->table = table;
  R->q1 = q1;
  R->q2 = q2;
  R->B = (int)B;
  R->U = (int)U;
  R->ncol = (int)ncol;
  R->n_rows = n_rows;
  R->p = to_params(params);
  R->ans_id = reinterpret_cast<const long long*>(ans_id);
  R->ans_count = ans_count;
  R->A = (int)A;
  return SMX_OK;
}

static int rank_run(int model, hipStream_t st, const RankArgs& R, int vec, int nit, int keys_only) {
  switch (model) {
    case mL1: return rank_dispatch<mL1>(st, R, vec, nit, keys_only);
    case mL2: return rank_dispatch<mL2>(st, R, vec, nit, keys_only);
    case mBox: return rank_dispatch<mBox>(st, R, vec, nit, keys_only);
    case mRotate: return rank_dispatch<mRotate>(st, R, vec, nit, keys_only);
    case mBetaKL: return rank_dispatch<mBetaKL>(st, R, vec, nit, keys_only);
    case mComplex: return rank_dispatch<mComplex>(st, R, vec, nit, keys_only);
    case mDistmult: return rank_dispatch<mDistmult>(st, R, vec, nit, keys_only);
  }
  return fail(SMX_ERR_KIND, "unknown score model %d", model);
}

}  // namespace smx

extern "C" {

size_t smx_rank_workspace_bytes(size_t B, size_t A) { return smx::rank_ws_bytes(B, A); }

int smx_rank_answer_keys_union(int model, void* stream, const float* table, size_t n_rows, const float* q1,
                               const float* q2, size_t B, size_t U, size_t dim, const smx_score_params* params,
                               const int64_t* ans_id, const int32_t* ans_count, size_t A, float* ans_score,
                               uint64_t* ans_key) {
  using namespace smx;
  RankArgs R;
  int vec, nit;
  if (int rc = rank_common(&R, &vec, &nit, model, table, n_rows, q1, q2, B, U, dim, params, ans_id, ans_count, A)) return rc;
  if (!ans_score || !ans_key) return fail(SMX_ERR_ARG, "null output pointer");
  R.score_out = ans_score;
  R.key_out = reinterpret_cast<unsigned long long*>(ans_key);
  return rank_run(model, as_stream(stream), R, vec, nit, kRankKeys);
}

int smx_rank_answer_keys(int model, void* stream, const float* table, size_t n_rows, const float* q1, const float* q2,
                         size_t B, size_t dim, const smx_score_params* params, const int64_t* ans_id,
                         const int32_t* ans_count, size_t A, float* ans_score, uint64_t* ans_key) {
  return smx_rank_answer_keys_union(model, stream, table, n_rows, q1, q2, B, 1, dim, params, ans_id, ans_count, A,
                                    ans_score, ans_key);
}

int smx_rank_scan_union(int model, void* stream, const float* table, size_t n_rows, const float* q1, const float* q2,
                        size_t B, size_t U, size_t dim, const smx_score_params* params, const int64_t* ans_id,
                        const uint64_t* ans_key, const int32_t* ans_count, size_t A, int64_t* filtered_rank,
                        void* workspace, size_t workspace_bytes) {
  using namespace smx;
  RankArgs R;
  int vec, nit;
  if (int rc = rank_common(&R, &vec, &nit, model, table, n_rows, q1, q2, B, U, dim, params, ans_id, ans_count, A)) return rc;
  if (!ans_key || !filtered_rank || !workspace) return fail(SMX_ERR_ARG, "null pointer");
  if (workspace_bytes < rank_ws_bytes(B, A))
    return fail(SMX_ERR_WORKSPACE, "rank workspace too small: %zu < %zu", workspace_bytes, rank_ws_bytes(B, A));
  R.ans_key = reinterpret_cast<const unsigned long long*>(ans_key);
  R.bins = static_cast<unsigned*>(workspace);
  R.rank_out = reinterpret_cast<long long*>(filtered_rank);
  return rank_run(model, as_stream(stream), R, vec, nit, kRankScan);
}

int smx_rank_scan(int model, void* stream, const float* table, size_t n_rows, const float* q1, const float* q2, size_t B,
                  size_t dim, const smx_score_params* params, const int64_t* ans_id, const uint64_t* ans_key,
                  const int32_t* ans_count, size_t A, int64_t* filtered_rank, void* workspace, size_t workspace_bytes) {
  return smx_rank_scan_union(model, stream, table, n_rows, q1, q2, B, 1, dim, params, ans_id, ans_key, ans_count, A,
                             filtered_rank, workspace, workspace_bytes);
}

int smx_rank_candidates_union(int model, void* stream, const float* table, size_t n_rows, const float* q1,
                              const float* q2, size_t B, size_t U, size_t dim, const smx_score_params* params,
                              const int64_t* cand, size_t C, const int32_t* n_hard, size_t H, float* logit,
                              int64_t* ranking, int64_t* hard_rank, int* err_flag) {
  using namespace smx;
  RankArgs R;
  int vec, nit;
  if (!cand || !n_hard || !ranking || !hard_rank) return fail(SMX_ERR_ARG, "null pointer");
  if (C == 0 || C > kRankMaxCandidates) return fail(SMX_ERR_SHAPE, "1 to %zu candidates per query", kRankMaxCandidates);
  if (H == 0 || H > C) return fail(SMX_ERR_SHAPE, "between 1 and C hard-answer slots");
  // (the shape checks shared with the all-entity scan; its answer arguments are not used here)
  if (int rc = rank_common(&R, &vec, &nit, model, table, n_rows, q1, q2, B, U, dim, params, cand, n_hard, 1)) return rc;
  if (B * C > 0x7fffffffull) return fail(SMX_ERR_SHAPE, "too many candidates in one call");
  R.ans_id = nullptr;
  R.ans_count = nullptr;
  R.cand = reinterpret_cast<const long long*>(cand);
  R.C = (int)C;
  R.H = (int)H;
  R.n_hard = n_hard;
  R.cand_logit = logit;
  R.cand_rank = reinterpret_cast<long long*>(ranking);
  R.hard_rank = reinterpret_cast<long long*>(hard_rank);
  R.err = err_flag;
  return rank_run(model, as_stream(stream), R, vec, nit, kRankCandidates);
}

int smx_rank_candidates(int model, void* stream, const float* table, size_t n_rows, const float* q1, const float* q2,
                        size_t B, size_t dim, const smx_score_params* params, const int64_t* cand, size_t C,
                        const int32_t* n_hard, size_t H, float* logit, int64_t* ranking, int64_t* hard_rank,
                        int* err_flag) {
  return smx_rank_candidates_union(model, stream, table, n_rows, q1, q2, B, 1, dim, params, cand, C, n_hard, H, logit,
                                   ranking, hard_rank, err_flag);
}

}  // extern "C"
