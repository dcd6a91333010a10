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
#include <algorithm>
#include <mutex>

#include "../../include/smx_measure.h"

#include "smx_score_impl.h"
#include "smx_shared_fwd_impl.h"

namespace smx {

extern template int score_dispatch<mL1>(hipStream_t, const ScoreArgs&, int, int, bool);
extern template int score_dispatch<mL2>(hipStream_t, const ScoreArgs&, int, int, bool);
extern template int score_dispatch<mBox>(hipStream_t, const ScoreArgs&, int, int, bool);
extern template int score_dispatch<mRotate>(hipStream_t, const ScoreArgs&, int, int, bool);
extern template int score_dispatch<mBetaKL>(hipStream_t, const ScoreArgs&, int, int, bool);
extern template int score_dispatch<mComplex>(hipStream_t, const ScoreArgs&, int, int, bool);
extern template int score_dispatch<mDistmult>(hipStream_t, const ScoreArgs&, int, int, bool);

// defined in smx_entity.hip
int entity_backward(int model, void* stream, const smx_plan_view* plan, float* table, size_t n_rows, const float* q1,
                    const float* q2, const float* score, const float* gscore, size_t B, size_t K, size_t dim,
                    const smx_score_params* params, float* merged, float* m, float* v, const smx_opt_params* adam,
                    void* workspace, size_t workspace_bytes, int skip_single, const unsigned char* codes, int codes_vec,
                    int codes_nit, const PairSources* multi = nullptr);
size_t entity_ws_bytes(size_t n_pairs, size_t row_len);
size_t code_bytes_per_pair(size_t dim);

// instantiated in smx_shared_inst_*.hip
extern template int shared_forward_dispatch<mL1>(hipStream_t, const SharedFwdArgs&, int);
extern template int shared_forward_dispatch<mL2>(hipStream_t, const SharedFwdArgs&, int);
extern template int shared_forward_dispatch<mBox>(hipStream_t, const SharedFwdArgs&, int);
extern template int shared_forward_dispatch<mRotate>(hipStream_t, const SharedFwdArgs&, int);

// defined in smx_shared_gemm.hip: shared negatives of beta_kl, complex and distmult as matrix products
size_t shared_gemm_workspace_floats(int model, size_t B, size_t K, size_t dim, bool entity, bool norm);
bool shared_gemm_fits(int model, size_t dim, const void* table, const void* q1, const void* q2, const void* workspace,
                      size_t workspace_bytes, size_t B, size_t K, bool entity, bool norm);
int shared_gemm_forward(int model, hipStream_t st, const float* table, size_t n_rows, const long long* ids,
                        const float* q1, const float* q2, float* score, size_t B, size_t K, size_t dim,
                        const ScoreParams& p, int* err, float* workspace);
int shared_list_rows(hipStream_t st, const float* table, size_t n_rows, const long long* ids, size_t K, size_t width,
                     float* out);
int shared_gemm_backward_query(int model, hipStream_t st, const float* table, size_t n_rows, const long long* ids,
                               const float* q1, const float* q2, const float* gscore, float* gq1, float* gq2, size_t B,
                               size_t K, size_t dim, const ScoreParams& p, float* workspace, size_t workspace_bytes);

// One extra stream and two events per device, created at first use and kept for the life of the process.
struct SideStream {
  hipStream_t stream = nullptr;
  hipEvent_t fork = nullptr, join = nullptr;
  std::mutex in_use;  // held while one call records, waits on and re-records the two events
};
static SideStream* side_stream() {
  static std::mutex mu;
  static SideStream per_device[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return nullptr;
  std::lock_guard<std::mutex> lock(mu);
  SideStream& s = per_device[dev];
  if (!s.stream) {
    hipStream_t st = nullptr;
    hipEvent_t f = nullptr, j = nullptr;
    if (hipStreamCreateWithFlags(&st, hipStreamNonBlocking) != hipSuccess) return nullptr;  // default priority
    if (hipEventCreateWithFlags(&f, hipEventDisableTiming) != hipSuccess ||
        hipEventCreateWithFlags(&j, hipEventDisableTiming) != hipSuccess)
      return nullptr;
    s.fork = f;
    s.join = j;
    s.stream = st;
  }
  return &s;
}

// Sign codes are laid out for float4 columns when dim is a multiple of 4, single floats otherwise, and
// exist for rows of up to 512 floats.  Returns null when (vec, nit) of this call fits that layout and
// the buffer has the size smx_score_codes_bytes gives, else what is wrong.
static const char* codes_mismatch(int model, size_t n_pairs, size_t dim, int vec, int nit, size_t codes_bytes) {
  if (!model_coded(model)) return "this model has no sign codes";
  if (vec != (dim % 4 == 0 ? 4 : 1)) return "sign codes need 16-byte aligned rows when dim is a multiple of 4";
  if (nit > 2) return "sign codes exist for rows of up to 512 floats";
  if (codes_bytes != n_pairs * code_bytes_per_pair(dim)) return "codes buffer is not smx_score_codes_bytes() long";
  return nullptr;
}

static int dispatch_model(int model, hipStream_t st, const ScoreArgs& A, int vec, int nit, bool forward) {
  switch (model) {
    case mL1: return score_dispatch<mL1>(st, A, vec, nit, forward);
    case mL2: return score_dispatch<mL2>(st, A, vec, nit, forward);
    case mBox: return score_dispatch<mBox>(st, A, vec, nit, forward);
    case mRotate: return score_dispatch<mRotate>(st, A, vec, nit, forward);
    case mBetaKL: return score_dispatch<mBetaKL>(st, A, vec, nit, forward);
    case mComplex: return score_dispatch<mComplex>(st, A, vec, nit, forward);
    case mDistmult: return score_dispatch<mDistmult>(st, A, vec, nit, forward);
  }
  return fail(SMX_ERR_KIND, "unknown score model %d", model);
}

// Where the rows finished by the query-gradient kernel go: table / optimizer state and/or merged rows.
static void fill_sink(ScoreArgs* A, float* table, float* m, float* v, float* merged, const smx_opt_params* adam) {
  A->sink.table = table;
  A->sink.m = m;
  A->sink.v = v;
  A->sink.merged = merged;
  A->sink.adam_on = adam ? adam->kind : 0;
  A->sink.squeeze = (adam && adam->squeeze) ? 1 : 0;
  if (adam) A->sink.a = make_adam_consts(adam);
  A->sink.step_dev = adam ? adam->step_consts_dev : nullptr;
  A->sink.p = A->p;
  A->sink.ncol = A->ncol;
}

// The step's query tensors do not fit one XCD's 4 MiB L2: the entity pass would fetch a one-pair
// segment's query rows from beyond it (measured: finishing such segments in the pair-ordered kernel is
// faster for 4096 queries x 2 x 200 floats, slower for 1024 queries x 2 x 400 or 500).
static bool queries_beyond_l2(int model, size_t B, size_t dim) {
  return B * dim * model_nq(model) * sizeof(float) > ((size_t)4 << 20);
}

// Common argument checks; fills the shape fields of A and picks the column width: float4 columns when
// rows are 16-byte aligned, single floats otherwise.
static int fill_args(ScoreArgs* A, int* vec, int* nit, int model, const float* table, size_t n_rows,
                     const int64_t* idx, const float* q1, const float* q2, size_t B, size_t K, size_t dim,
                     const smx_score_params* params, const void* extra_a, const void* extra_b) {
  if (model < 0 || model >= mNumModels) return fail(SMX_ERR_KIND, "unknown score model %d", model);
  if (!table || !q1 || !params || (model_nq(model) == 2 && !q2)) return fail(SMX_ERR_ARG, "null pointer");
  if (B == 0 || K == 0 || dim == 0) return fail(SMX_ERR_SHAPE, "empty dimension");
  if (B > 0x7fffffffull || K > 0x7fffffffull || B * K > 0x7fffffffull)
    return fail(SMX_ERR_SHAPE, "more than 2^31-1 pairs in one call");
  if (idx && n_rows > 0xffffffffull)  // the kernels tell ids apart by their low 32 bits, as the segment plan does
    return fail(SMX_ERR_SHAPE, "entity count %zu needs ids wider than 32 bits", n_rows);
  if (const char* why = params_refused(model, params)) return fail(SMX_ERR_ARG, "%s", why);
  const bool vec4 = dim % 4 == 0 && aligned16(table) && aligned16(q1) && (model_nq(model) == 1 || aligned16(q2)) &&
                    aligned16(extra_a) && aligned16(extra_b);
  *vec = vec4 ? 4 : 1;
  const size_t ncol = dim / *vec;
  const int need = (int)((ncol + 63) / 64);
  *nit = need <= 1 ? 1 : (need <= 2 ? 2 : (need <= 4 ? 4 : 8));
  if (ncol > 512 || (*vec == 1 && *nit > 4))
    return fail(SMX_ERR_SHAPE, "dim %zu not supported by the fused path (at most 2048 aligned or 256 unaligned floats)", dim);
  *A = ScoreArgs{};
  A->table = table;
  A->idx = reinterpret_cast<const long long*>(idx);
  A->q1 = q1;
  A->q2 = q2;
  A->B = (int)B;
  A->K = (int)K;
  A->ncol = (int)ncol;
  A->n_rows = idx ? n_rows : B * K;
  A->U = 1;
  A->p = to_params(params);
  return SMX_OK;
}

// score[b,k] = max over the branches u of branch[b*U+u, k], winner[b,k] = the first branch that holds it -- what
// torch.max(logit, dim=1) returns as values and indices in the custom_cal_logit bodies (box.py:163).
__global__ __launch_bounds__(256) void union_max_kernel(const float* __restrict__ branch, float* __restrict__ score,
                                                        unsigned char* __restrict__ winner, int U, int K, size_t n) {
  const size_t p = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (p >= n) return;
  const size_t b = p / K, k = p - b * K;
  float best = branch[(b * U) * K + k];
  int at = 0;
  for (int u = 1; u < U; ++u) {
    const float s = branch[(b * U + u) * K + k];
    if (s > best || (s != s && best == best)) {  // torch.max: a NaN wins, and the first of equals stays
      best = s;
      at = u;
    }
  }
  score[p] = best;
  winner[p] = (unsigned char)at;
}

}  // namespace smx

extern "C" {

size_t smx_score_codes_bytes(int model, size_t n_pairs, size_t dim) {
  using namespace smx;
  if (model < 0 || model >= mNumModels || !model_coded(model)) return 0;
  const size_t per_pair = code_bytes_per_pair(dim);
  return per_pair > 2 * 64 ? 0 : n_pairs * per_pair;
}

int smx_score_forward(int model, void* stream, const float* table, size_t n_rows, const int64_t* idx,
                      const float* q1, const float* q2, float* score, size_t B, size_t K, size_t dim,
                      const smx_score_params* params, int* err_flag, void* codes, size_t codes_bytes) {
  using namespace smx;
  ScoreArgs A;
  int vec, nit;
  if (int rc = fill_args(&A, &vec, &nit, model, table, n_rows, idx, q1, q2, B, K, dim, params, nullptr, nullptr)) return rc;
  if (!score) return fail(SMX_ERR_ARG, "null score pointer");
  if (codes) {
    if (const char* msg = codes_mismatch(model, B * K, dim, vec, nit, codes_bytes)) return fail(SMX_ERR_ARG, "%s", msg);
    if (reinterpret_cast<uintptr_t>(codes) & 15u) return fail(SMX_ERR_ARG, "codes must be 16-byte aligned");
    A.codes = static_cast<unsigned char*>(codes);
  }
  A.score_out = score;
  A.err = err_flag;
  return dispatch_model(model, as_stream(stream), A, vec, nit, true);
}

int smx_score_backward_query(int model, void* stream, const float* table, size_t n_rows, const int64_t* idx,
                             const float* q1, const float* q2, const float* score, const float* gscore, float* gq1,
                             float* gq2, size_t B, size_t K, size_t dim, const smx_score_params* params,
                             const void* fwd_codes, size_t fwd_codes_bytes) {
  using namespace smx;
  ScoreArgs A;
  int vec, nit;
  if (int rc = fill_args(&A, &vec, &nit, model, table, n_rows, idx, q1, q2, B, K, dim, params, nullptr, nullptr)) return rc;
  if (!score || !gscore || !gq1 || (model_nq(model) == 2 && !gq2)) return fail(SMX_ERR_ARG, "null pointer");
  if (fwd_codes) {
    if (const char* msg = codes_mismatch(model, B * K, dim, vec, nit, fwd_codes_bytes)) return fail(SMX_ERR_ARG, "%s", msg);
    if (reinterpret_cast<uintptr_t>(fwd_codes) & 15u) return fail(SMX_ERR_ARG, "codes must be 16-byte aligned");
    A.codes_in = static_cast<const unsigned char*>(fwd_codes);
  }
  A.score = score;
  A.gscore = gscore;
  A.gq1 = gq1;
  A.gq2 = gq2;
  return dispatch_model(model, as_stream(stream), A, vec, nit, false);
}

size_t smx_shared_workspace_bytes(int model, size_t B, size_t K, size_t dim) {
  if (model < 0 || model >= smx::mNumModels) return 0;
  const size_t a = smx::shared_gemm_workspace_floats(model, B, K, dim, false, true);
  const size_t b = smx::shared_gemm_workspace_floats(model, B, K, dim, true, true);
  const size_t rows = K * smx::model_mul(model) * dim;  // the list's rows side by side (query backward)
  const size_t n = std::max(rows, std::max(a, b));
  return n ? ((n * sizeof(float) + 255) & ~(size_t)255) : 0;
}

int smx_score_forward_shared(int model, void* stream, const float* table, size_t n_rows, const int64_t* ids,
                             const float* q1, const float* q2, float* score, size_t B, size_t K, size_t dim,
                             const smx_score_params* params, int* err_flag, void* workspace, size_t workspace_bytes) {
  using namespace smx;
  ScoreArgs A;
  int vec, nit;
  if (!ids) return fail(SMX_ERR_ARG, "null id list");
  if (int rc = fill_args(&A, &vec, &nit, model, table, n_rows, ids, q1, q2, B, K, dim, params, nullptr, nullptr)) return rc;
  if (!score) return fail(SMX_ERR_ARG, "null score pointer");
  // BetaE (the entity side of the divergence once per shared row: needs the workspace), ComplEx, DistMult: the pairs
  // as a matrix product
  if (shared_gemm_fits(model, dim, table, q1, q2, workspace, workspace_bytes, B, K, false, A.p.norm_on != 0))
    return shared_gemm_forward(model, as_stream(stream), table, n_rows, reinterpret_cast<const long long*>(ids), q1, q2,
                               score, B, K, dim, A.p, err_flag, static_cast<float*>(workspace));
  if (shared_forward_fits(model, vec, nit)) {  // rows staged in LDS for eight queries at a time
    const SharedFwdArgs S{table, reinterpret_cast<const long long*>(ids), q1, q2, score, (int)B, (int)K, A.ncol, n_rows, A.p,
                          err_flag};
    hipStream_t st = as_stream(stream);
    switch (model) {
      case mL1: return shared_forward_dispatch<mL1>(st, S, nit);
      case mL2: return shared_forward_dispatch<mL2>(st, S, nit);
      case mBox: return shared_forward_dispatch<mBox>(st, S, nit);
      case mRotate: return shared_forward_dispatch<mRotate>(st, S, nit);
    }
  }
  A.ids_shared = 1;
  A.score_out = score;
  A.err = err_flag;
  return dispatch_model(model, as_stream(stream), A, vec, nit, true);
}

int smx_score_backward_query_shared(int model, void* stream, const float* table, size_t n_rows, const int64_t* ids,
                                    const float* q1, const float* q2, const float* score, const float* gscore,
                                    float* gq1, float* gq2, size_t B, size_t K, size_t dim,
                                    const smx_score_params* params, void* workspace, size_t workspace_bytes) {
  using namespace smx;
  ScoreArgs A;
  int vec, nit;
  if (!ids) return fail(SMX_ERR_ARG, "null id list");
  if (int rc = fill_args(&A, &vec, &nit, model, table, n_rows, ids, q1, q2, B, K, dim, params, nullptr, nullptr)) return rc;
  if (!score || !gscore || !gq1 || (model_nq(model) == 2 && !gq2)) return fail(SMX_ERR_ARG, "null pointer");
  if (shared_gemm_fits(model, dim, table, q1, q2, workspace, workspace_bytes, B, K, false, A.p.norm_on != 0))
    return shared_gemm_backward_query(model, as_stream(stream), table, n_rows, reinterpret_cast<const long long*>(ids), q1,
                                      q2, gscore, gq1, gq2, B, K, dim, A.p, static_cast<float*>(workspace), workspace_bytes);
  A.ids_shared = 1;
  // Every query's workgroup reads all K rows.  Out of a table of many gigabytes those are K scattered pages,
  // translated again by each of them; copied side by side first (one small launch) they are one stretch of memory
  // that stays in L2.  B = 512, K = 1024, D = 400, box: the copy costs 5 us and the kernel then takes 57 whatever
  // the table's size, against 55 / 59 / 65 / 69 / 75 us from a table of 3 / 6 / 16 / 32 / 64 GB.
  const size_t width = (size_t)model_mul(model) * dim;
  const bool far_apart = n_rows * width * sizeof(float) >= ((size_t)8 << 30);
  if (far_apart && workspace && aligned16(workspace) && vec == 4 && workspace_bytes >= K * width * sizeof(float) &&
      K >= 64 && B >= 16) {
    float* rows = static_cast<float*>(workspace);
    if (int rc = shared_list_rows(as_stream(stream), table, n_rows, reinterpret_cast<const long long*>(ids), K, width, rows))
      return rc;
    A.table = rows;
    A.idx = nullptr;   // row k of the copy is list position k
    A.n_rows = K;
  }
  A.score = score;
  A.gscore = gscore;
  A.gq1 = gq1;
  A.gq2 = gq2;
  return dispatch_model(model, as_stream(stream), A, vec, nit, false);
}

size_t smx_union_workspace_bytes(size_t B, size_t U, size_t K) { return (B * U * K * sizeof(float) + 255) & ~(size_t)255; }

int smx_score_forward_union(int model, void* stream, const float* table, size_t n_rows, const int64_t* idx,
                            const float* q1, const float* q2, float* score, uint8_t* winner, size_t B, size_t U,
                            size_t K, size_t dim, const smx_score_params* params, int* err_flag, void* workspace,
                            size_t workspace_bytes) {
  using namespace smx;
  ScoreArgs A;
  int vec, nit;
  if (!idx) return fail(SMX_ERR_ARG, "null id tensor");
  if (U == 0 || U > 255) return fail(SMX_ERR_SHAPE, "1 to 255 union branches");
  if (B > 0x7fffffffull / U) return fail(SMX_ERR_SHAPE, "too many branch rows");
  if (int rc = fill_args(&A, &vec, &nit, model, table, n_rows, idx, q1, q2, B * U, K, dim, params, nullptr, nullptr)) return rc;
  if (!score || !winner) return fail(SMX_ERR_ARG, "null output pointer");
  if (!workspace || (reinterpret_cast<uintptr_t>(workspace) & 15u) || workspace_bytes < smx_union_workspace_bytes(B, U, K))
    return fail(SMX_ERR_WORKSPACE, "the union forward needs smx_union_workspace_bytes() of 16-byte aligned workspace");
  A.U = (int)U;
  A.score_out = static_cast<float*>(workspace);  // [B*U, K]: every branch's logits
  A.err = err_flag;
  hipStream_t st = as_stream(stream);
  if (int rc = dispatch_model(model, st, A, vec, nit, true)) return rc;
  const size_t n = B * K;
  hipLaunchKernelGGL(union_max_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, A.score_out, score, winner,
                     (int)U, (int)K, n);
  return check_launch("union maximum");
}

int smx_score_backward_query_union(int model, void* stream, const float* table, size_t n_rows, const int64_t* idx,
                                   const float* q1, const float* q2, const float* score, const float* gscore,
                                   const uint8_t* winner, float* gq1, float* gq2, size_t B, size_t U, size_t K,
                                   size_t dim, const smx_score_params* params) {
  using namespace smx;
  ScoreArgs A;
  int vec, nit;
  if (!idx) return fail(SMX_ERR_ARG, "null id tensor");
  if (U == 0 || U > 255) return fail(SMX_ERR_SHAPE, "1 to 255 union branches");
  if (B > 0x7fffffffull / U) return fail(SMX_ERR_SHAPE, "too many branch rows");
  if (int rc = fill_args(&A, &vec, &nit, model, table, n_rows, idx, q1, q2, B * U, K, dim, params, nullptr, nullptr)) return rc;
  if (!score || !gscore || !winner || !gq1 || (model_nq(model) == 2 && !gq2)) return fail(SMX_ERR_ARG, "null pointer");
  A.U = (int)U;
  A.winner = winner;
  A.score = score;
  A.gscore = gscore;
  A.gq1 = gq1;
  A.gq2 = gq2;
  return dispatch_model(model, as_stream(stream), A, vec, nit, false);
}

int smx_score_backward_entity(int model, void* stream, const smx_plan_view* plan, float* table, size_t n_rows,
                              const float* q1, const float* q2, const float* score, const float* gscore, size_t B,
                              size_t K, size_t dim, const smx_score_params* params, float* merged, float* m, float* v,
                              const smx_opt_params* adam, void* workspace, size_t workspace_bytes,
                              const void* fwd_codes, size_t fwd_codes_bytes) {
  using namespace smx;
  int codes_vec = 0, codes_nit = 0;
  if (fwd_codes) {
    // the layout smx_score_codes_bytes promises; entity_backward refuses the call if its own column
    // layout (alignment of merged / m / v included) turns out different
    if (model < 0 || model >= mNumModels || !model_coded(model)) return fail(SMX_ERR_ARG, "this model has no sign codes");
    if (fwd_codes_bytes != B * K * code_bytes_per_pair(dim) || code_bytes_per_pair(dim) > 2 * 64)
      return fail(SMX_ERR_ARG, "codes buffer is not smx_score_codes_bytes() long");
    if (reinterpret_cast<uintptr_t>(fwd_codes) & 15u) return fail(SMX_ERR_ARG, "codes must be 16-byte aligned");
    codes_vec = dim % 4 == 0 ? 4 : 1;
    codes_nit = (int)(code_bytes_per_pair(dim) / 64);
  }
  const unsigned char* codes = static_cast<const unsigned char*>(fwd_codes);
  // Large steps with the forward's codes and an optimizer: the one-pair segments (most of the touched
  // rows of a skewed or sparse id stream) go through the pair-ordered kernel on the caller's stream while
  // the entity pass reduces the others on the library's second stream -- the same division of work and
  // the same arithmetic per row as in smx_score_backward_fused, minus the query gradient.
  // (everything the entity pass would refuse is checked here first, so that a refused call has not
  // already updated the one-pair rows)
  const bool split = fwd_codes && adam && !merged && plan && plan->pair_seg && plan->uniq && plan->order &&
                     plan->sorted_ids && plan->seg_of_pos && plan->seg_start && plan->n_uniq && score && gscore &&
                     queries_beyond_l2(model, B, dim) && B * K >= ((size_t)1 << 20) && plan->n_pairs == B * K &&
                     workspace && !(reinterpret_cast<uintptr_t>(workspace) & 255u) &&
                     workspace_bytes >= entity_ws_bytes(B * K, dim * model_mul(model)) &&
                     !serial_backward();
  if (split) {
    ScoreArgs A;
    int vec, nit;
    if (const char* msg = check_opt_params(adam, m, v)) return fail(SMX_ERR_ARG, "%s", msg);
    if (int rc = fill_args(&A, &vec, &nit, model, table, n_rows, nullptr, q1, q2, B, K, dim, params, nullptr, m)) return rc;
    const bool v_ok = !(vec == 4 && v && !adam->squeeze && !aligned16(v));
    if (vec == codes_vec && nit == codes_nit && v_ok) {
      A.n_rows = n_rows;
      A.score = score;
      A.gscore = gscore;
      A.pair_seg = plan->pair_seg;
      A.uniq = reinterpret_cast<const long long*>(plan->uniq);
      fill_sink(&A, table, m, v, nullptr, adam);
      SideStream* side = side_stream();
      if (!side) return fail(SMX_ERR_HIP, "cannot create the side stream");
      hipStream_t st = as_stream(stream);
      std::lock_guard<std::mutex> one_call(side->in_use);
      if (hipEventRecord(side->fork, st) != hipSuccess || hipStreamWaitEvent(side->stream, side->fork, 0) != hipSuccess)
        return fail(SMX_ERR_HIP, "fork to the side stream failed");
      int rc = dispatch_model(model, st, A, vec, nit, false);  // gq1 == null: one-pair segments only
      if (rc == SMX_OK)
        rc = entity_backward(model, side->stream, plan, table, n_rows, q1, q2, score, gscore, B, K, dim, params, nullptr,
                             m, v, adam, workspace, workspace_bytes, 1, codes, codes_vec, codes_nit);
      if (hipEventRecord(side->join, side->stream) != hipSuccess || hipStreamWaitEvent(st, side->join, 0) != hipSuccess)
        return fail(SMX_ERR_HIP, "join with the side stream failed");
      return rc;
    }
  }
  return entity_backward(model, stream, plan, table, n_rows, q1, q2, score, gscore, B, K, dim, params, merged, m, v,
                         adam, workspace, workspace_bytes, 0, codes, codes_vec, codes_nit);
}

}  // extern "C"

namespace smx {

// U: branch rows per query in q1 / q2 (union queries); 1 for every caller but smx_score_backward_entity_union
static int entity_multi(int model, void* stream, const smx_plan_view* plan, float* table, size_t n_rows,
                        const float* q1, const float* q2, const smx_pair_source* src, size_t n_src,
                        size_t B, size_t U, size_t dim, const smx_score_params* params, float* merged, float* m,
                        float* v, const smx_opt_params* adam, void* workspace, size_t workspace_bytes,
                        const float* grad_rows, size_t n_grad_rows) {
  if (!src || n_src == 0 || n_src > (size_t)kMaxSources)
    return fail(SMX_ERR_ARG, "1 to %d pair sources", kMaxSources);
  if ((grad_rows != nullptr) != (n_grad_rows != 0)) return fail(SMX_ERR_ARG, "gradient rows and their count must come together");
  if (U == 0 || U > 255) return fail(SMX_ERR_SHAPE, "1 to 255 union branches");
  if (n_src == 1 && (src[0].q_first != 0 || (src[0].n_queries != 0 && src[0].n_queries != B)))
    return fail(SMX_ERR_ARG, "a single pair source covers all B queries");
  if (n_src == 1 && !grad_rows && U == 1)
    return smx_score_backward_entity(model, stream, plan, table, n_rows, q1, q2, src[0].score, src[0].gscore, B,
                                     src[0].K, dim, params, merged, m, v, adam, workspace, workspace_bytes,
                                     src[0].fwd_codes, src[0].fwd_codes_bytes);
  if (model < 0 || model >= mNumModels) return fail(SMX_ERR_KIND, "unknown score model %d", model);
  PairSources S{};
  S.n = (int)n_src;
  size_t k_sum = 0, n_model = 0;
  const bool coded = src[0].fwd_codes != nullptr;
  int codes_vec = 0, codes_nit = 0;
  if (coded) {
    if (!model_coded(model) || code_bytes_per_pair(dim) > 2 * 64) return fail(SMX_ERR_ARG, "this model has no sign codes");
    codes_vec = dim % 4 == 0 ? 4 : 1;
    codes_nit = (int)(code_bytes_per_pair(dim) / 64);
  }
  for (size_t i = 0; i < n_src; ++i) {
    if (!src[i].score || !src[i].gscore || src[i].K == 0) return fail(SMX_ERR_ARG, "incomplete pair source %zu", i);
    if ((src[i].fwd_codes != nullptr) != coded) return fail(SMX_ERR_ARG, "sign codes for some pair sources only");
    if (coded) {
      if (src[i].fwd_codes_bytes != (src[i].n_queries ? src[i].n_queries : B) * src[i].K * code_bytes_per_pair(dim))
        return fail(SMX_ERR_ARG, "codes buffer of source %zu is not smx_score_codes_bytes() long", i);
      if (reinterpret_cast<uintptr_t>(src[i].fwd_codes) & 15u) return fail(SMX_ERR_ARG, "codes must be 16-byte aligned");
    }
    S.score[i] = src[i].score;
    S.gscore[i] = src[i].gscore;
    S.codes[i] = static_cast<const unsigned char*>(src[i].fwd_codes);
    S.K[i] = src[i].K;
    S.B[i] = src[i].n_queries ? src[i].n_queries : B;
    S.q_first[i] = src[i].q_first;
    if (S.q_first[i] + S.B[i] > B)
      return fail(SMX_ERR_SHAPE, "pair source %zu: queries %zu .. %zu of %zu", i, S.q_first[i], S.q_first[i] + S.B[i], B);
    S.winner[i] = src[i].winner;
    if (U > 1 && !src[i].winner) return fail(SMX_ERR_ARG, "union queries: pair source %zu has no winner array", i);
    k_sum += src[i].K;
    n_model += S.B[i] * src[i].K;
  }
  S.U = U;
  if (U > 1 && coded) return fail(SMX_ERR_ARG, "union queries have no sign codes");
  S.grad_rows = grad_rows;
  S.n_grad = n_grad_rows;
  const size_t n_all = n_model + n_grad_rows;
  if (B == 0 || n_all > 0x7fffffffull) return fail(SMX_ERR_SHAPE, "pair count out of range");
  if (!plan || plan->n_pairs != n_all)
    return fail(SMX_ERR_SHAPE, "the plan must hold the %zu pairs of all sources and the %zu gradient rows", n_model,
                n_grad_rows);
  // the same division of work as smx_score_backward_entity: ids that occur once in the whole step go through
  // the pair-ordered kernel, one launch per source, while the entity pass reduces the others beside it
  const bool split = coded && adam && !merged && plan->pair_seg && plan->uniq && plan->order && plan->sorted_ids &&
                     plan->seg_of_pos && plan->seg_start && plan->n_uniq && queries_beyond_l2(model, B, dim) &&
                     n_model >= ((size_t)1 << 20) && workspace && !(reinterpret_cast<uintptr_t>(workspace) & 255u) &&
                     workspace_bytes >= entity_ws_bytes(n_all, dim * model_mul(model)) && !serial_backward() &&
                     (!grad_rows || aligned16(grad_rows));
  if (split) {
    if (const char* msg = check_opt_params(adam, m, v)) return fail(SMX_ERR_ARG, "%s", msg);
    ScoreArgs A[kMaxSources];
    bool fits = true;
    size_t first = 0;
    for (size_t i = 0; i < n_src && fits; ++i) {
      int vec, nit;
      // (the one-pair kernel numbers a source's queries from its own first row)
      const float* s_q1 = q1 + S.q_first[i] * dim;
      const float* s_q2 = q2 ? q2 + S.q_first[i] * dim : nullptr;
      if (int rc = fill_args(&A[i], &vec, &nit, model, table, n_rows, nullptr, s_q1, s_q2, S.B[i], src[i].K, dim, params,
                             nullptr, m))
        return rc;
      fits = vec == codes_vec && nit == codes_nit && !(vec == 4 && v && !adam->squeeze && !aligned16(v));
      A[i].n_rows = n_rows;
      A[i].score = src[i].score;
      A[i].gscore = src[i].gscore;
      A[i].codes_in = S.codes[i];
      A[i].pair_seg = plan->pair_seg + first;
      A[i].uniq = reinterpret_cast<const long long*>(plan->uniq);
      fill_sink(&A[i], table, m, v, nullptr, adam);
      first += S.B[i] * src[i].K;
    }
    if (fits) {
      SideStream* side = side_stream();
      if (!side) return fail(SMX_ERR_HIP, "cannot create the side stream");
      hipStream_t st = as_stream(stream);
      std::lock_guard<std::mutex> one_call(side->in_use);
      if (hipEventRecord(side->fork, st) != hipSuccess || hipStreamWaitEvent(side->stream, side->fork, 0) != hipSuccess)
        return fail(SMX_ERR_HIP, "fork to the side stream failed");
      int rc = SMX_OK;
      for (size_t i = 0; i < n_src && rc == SMX_OK; ++i)
        rc = dispatch_model(model, st, A[i], codes_vec, codes_nit, false);  // gq1 == null: one-pair segments only
      if (rc == SMX_OK)
        rc = entity_backward(model, side->stream, plan, table, n_rows, q1, q2, nullptr, nullptr, B, k_sum, dim, params,
                             nullptr, m, v, adam, workspace, workspace_bytes, 1, S.codes[0], codes_vec, codes_nit, &S);
      if (hipEventRecord(side->join, side->stream) != hipSuccess || hipStreamWaitEvent(st, side->join, 0) != hipSuccess)
        return fail(SMX_ERR_HIP, "join with the side stream failed");
      return rc;
    }
  }
  return entity_backward(model, stream, plan, table, n_rows, q1, q2, nullptr, nullptr, B, k_sum, dim, params, merged, m, v,
                         adam, workspace, workspace_bytes, 0, S.codes[0], codes_vec, codes_nit, &S);
}

}  // namespace smx

extern "C" {

int smx_score_backward_entity_multi(int model, void* stream, const smx_plan_view* plan, float* table, size_t n_rows,
                                    const float* q1, const float* q2, const smx_pair_source* src, size_t n_src,
                                    size_t B, size_t dim, const smx_score_params* params, float* merged, float* m,
                                    float* v, const smx_opt_params* adam, void* workspace, size_t workspace_bytes,
                                    const float* grad_rows, size_t n_grad_rows) {
  return smx::entity_multi(model, stream, plan, table, n_rows, q1, q2, src, n_src, B, 1, dim, params, merged, m, v, adam,
                           workspace, workspace_bytes, grad_rows, n_grad_rows);
}

int smx_score_backward_entity_union(int model, void* stream, const smx_plan_view* plan, float* table, size_t n_rows,
                                    const float* q1, const float* q2, const smx_pair_source* src, size_t n_src,
                                    size_t B, size_t U, size_t dim, const smx_score_params* params, float* merged,
                                    float* m, float* v, const smx_opt_params* adam, void* workspace,
                                    size_t workspace_bytes, const float* grad_rows, size_t n_grad_rows) {
  return smx::entity_multi(model, stream, plan, table, n_rows, q1, q2, src, n_src, B, U, dim, params, merged, m, v, adam,
                           workspace, workspace_bytes, grad_rows, n_grad_rows);
}

}  // extern "C"

namespace smx {

// parts: bit 0 the query-gradient kernel, bit 1 the entity pass (3 for every caller but the measuring entry point)
// smx_measure_query_kernel_events: the pair the next backward call of this thread records around its query kernel
static thread_local hipEvent_t g_query_before = nullptr, g_query_after = nullptr;

static int dispatch_query_kernel(int model, hipStream_t st, const ScoreArgs& A, int vec, int nit) {
  hipEvent_t before = g_query_before, after = g_query_after;
  g_query_before = g_query_after = nullptr;
  if (before && hipEventRecord(before, st) != hipSuccess) return fail(SMX_ERR_HIP, "cannot record the measuring event");
  const int rc = dispatch_model(model, st, A, vec, nit, false);
  if (after && hipEventRecord(after, st) != hipSuccess) return fail(SMX_ERR_HIP, "cannot record the measuring event");
  return rc;
}

static int backward_fused(int parts, int model, void* stream, const smx_plan_view* plan, float* table, size_t n_rows,
                          const int64_t* idx, const float* q1, const float* q2, const float* score,
                          const float* gscore, float* gq1, float* gq2, size_t B, size_t K, size_t dim,
                          const smx_score_params* params, float* merged, float* m, float* v,
                          const smx_opt_params* adam, void* workspace, size_t workspace_bytes,
                          const void* fwd_codes, size_t fwd_codes_bytes) {
  ScoreArgs A;
  int vec, nit;
  if (!idx) return fail(SMX_ERR_ARG, "the fused backward needs the id tensor");
  if (!plan || !plan->pair_seg) return fail(SMX_ERR_ARG, "the fused backward needs a plan built with pair_seg");
  if (plan->n_pairs != B * K) return fail(SMX_ERR_SHAPE, "plan holds %zu pairs, call has %zu", plan->n_pairs, B * K);
  if (!merged && !adam) return fail(SMX_ERR_ARG, "nothing to do: neither merged gradient nor an optimizer requested");
  if (!adam && (m || v)) return fail(SMX_ERR_ARG, "optimizer state given without optimizer parameters");
  if (adam)
    if (const char* msg = check_opt_params(adam, m, v)) return fail(SMX_ERR_ARG, "%s", msg);
  // the same column width must suit the query-backward kernel and the entity pass
  if (int rc = fill_args(&A, &vec, &nit, model, table, n_rows, idx, q1, q2, B, K, dim, params, merged, m)) return rc;
  if (vec == 4 && v && !(adam && adam->squeeze) && !aligned16(v))
    return fail(SMX_ERR_ARG, "v must be 16-byte aligned like the table");
  if (!score || !gscore || !gq1 || (model_nq(model) == 2 && !gq2)) return fail(SMX_ERR_ARG, "null pointer");
  // what the entity pass would refuse, before the query-gradient kernel has touched any row
  if (!plan->order || !plan->sorted_ids || !plan->seg_of_pos || !plan->seg_start || !plan->uniq || !plan->n_uniq)
    return fail(SMX_ERR_ARG, "incomplete segment plan");
  if (!workspace || (reinterpret_cast<uintptr_t>(workspace) & 255u))
    return fail(SMX_ERR_ARG, "workspace must be given and 256-byte aligned");
  if (workspace_bytes < entity_ws_bytes(B * K, dim * model_mul(model)))
    return fail(SMX_ERR_WORKSPACE, "fused workspace too small: %zu < %zu", workspace_bytes,
                entity_ws_bytes(B * K, dim * model_mul(model)));
  A.score = score;
  A.gscore = gscore;
  A.gq1 = gq1;
  A.gq2 = gq2;
  // Finishing one-pair segments in the query-gradient kernel pays when the entity pass would have to
  // fetch their query rows from beyond the L2: that is when the query tensors of the step are larger
  // than one XCD's 4 MiB L2 (measured: faster for 4096 queries x 2 x 200 floats, slower for 1024
  // queries x 2 x 400 or 500).  Otherwise every segment goes through the entity pass.
  // Without an optimizer the one-pair rows cost the query-gradient kernel one store each (nothing to
  // fetch), so they are always finished there.
  const bool q_beyond_l2 = queries_beyond_l2(model, B, dim);
  const bool singles_here = !adam || q_beyond_l2;
  A.pair_seg = singles_here ? plan->pair_seg : nullptr;
  fill_sink(&A, table, m, v, merged, adam);
  // Sign codes (models that have them): when the entity pass would fetch query rows from beyond the L2,
  // the query-gradient kernel leaves each pair's derivative decisions in the workspace behind the
  // entity pass's own scratch, and the entity pass reads those instead of the query rows.  Used when
  // the caller's workspace has the room (smx_fused_workspace_bytes).
  const unsigned char* codes = nullptr;
  if (fwd_codes) {
    // the forward pass left the codes: neither the query-gradient kernel nor the entity pass needs the
    // entity rows or the query rows for the derivative
    if (const char* msg = codes_mismatch(model, B * K, dim, vec, nit, fwd_codes_bytes)) return fail(SMX_ERR_ARG, "%s", msg);
    if (reinterpret_cast<uintptr_t>(fwd_codes) & 15u) return fail(SMX_ERR_ARG, "codes must be 16-byte aligned");
    A.codes_in = static_cast<const unsigned char*>(fwd_codes);
    codes = A.codes_in;
  } else if (model_coded(model) && q_beyond_l2 && workspace && nit <= 2) {  // rows of up to 512 floats
    const size_t base = entity_ws_bytes(B * K, dim * model_mul(model));
    const size_t need = (size_t)B * K * nit * 64;
    if (workspace_bytes >= base + need) {
      A.codes = static_cast<unsigned char*>(workspace) + base;
      codes = A.codes;
    }
  }
  // (the serial-backward option keeps everything on the caller's stream, for per-kernel profiling)
  if (fwd_codes && adam && B * K >= ((size_t)1 << 20) && !serial_backward()) {
    // With the forward's codes the entity pass does not depend on the query-gradient kernel and the two
    // touch disjoint rows; one is bound by instruction issue for much of its time, the other by memory
    // latency, so they run side by side: the entity pass on a second stream of the same device, forked
    // from and joined to the caller's stream with events.  Measured: 0.1 ms of 1.0 ms on the 86M-row
    // workload with Adam; no gain for the recomputing models or without optimizer, and the fork/join
    // costs ~40 us, which small steps do not earn back.
    SideStream* side = side_stream();
    if (!side) return fail(SMX_ERR_HIP, "cannot create the side stream");
    hipStream_t st = as_stream(stream);
    // two host threads on one device share the stream and its events: one fork .. join sequence at a time
    std::lock_guard<std::mutex> one_call(side->in_use);
    if (hipEventRecord(side->fork, st) != hipSuccess || hipStreamWaitEvent(side->stream, side->fork, 0) != hipSuccess)
      return fail(SMX_ERR_HIP, "fork to the side stream failed");
    int rc = (parts & 1) ? dispatch_query_kernel(model, st, A, vec, nit) : SMX_OK;
    if (rc == SMX_OK && (parts & 2))
      rc = entity_backward(model, side->stream, plan, table, n_rows, q1, q2, score, gscore, B, K, dim, params, merged, m,
                           v, adam, workspace, workspace_bytes, singles_here ? 1 : 0, codes, vec, nit);
    // join even after a failed launch, so that the caller's stream never runs ahead of the side stream
    if (hipEventRecord(side->join, side->stream) != hipSuccess || hipStreamWaitEvent(st, side->join, 0) != hipSuccess)
      return fail(SMX_ERR_HIP, "join with the side stream failed");
    return rc;
  }
  if (parts & 1)
    if (int rc = dispatch_query_kernel(model, as_stream(stream), A, vec, nit)) return rc;
  if (!(parts & 2)) return SMX_OK;
  return entity_backward(model, stream, plan, table, n_rows, q1, q2, score, gscore, B, K, dim, params, merged, m, v,
                         adam, workspace, workspace_bytes, singles_here ? 1 : 0, codes, vec, nit);
}

}  // namespace smx

extern "C" {

int smx_score_backward_fused(int model, void* stream, const smx_plan_view* plan, float* table, size_t n_rows,
                             const int64_t* idx, const float* q1, const float* q2, const float* score,
                             const float* gscore, float* gq1, float* gq2, size_t B, size_t K, size_t dim,
                             const smx_score_params* params, float* merged, float* m, float* v,
                             const smx_opt_params* adam, void* workspace, size_t workspace_bytes,
                             const void* fwd_codes, size_t fwd_codes_bytes) {
  return smx::backward_fused(3, model, stream, plan, table, n_rows, idx, q1, q2, score, gscore, gq1, gq2, B, K, dim, params,
                             merged, m, v, adam, workspace, workspace_bytes, fwd_codes, fwd_codes_bytes);
}

int smx_measure_query_kernel_events(void* before, void* after) {
  if ((before == nullptr) != (after == nullptr)) return smx::fail(SMX_ERR_ARG, "two events, or none");
  smx::g_query_before = static_cast<hipEvent_t>(before);
  smx::g_query_after = static_cast<hipEvent_t>(after);
  return SMX_OK;
}

int smx_measure_backward_fused(int parts, int model, void* stream, const smx_plan_view* plan, float* table, size_t n_rows,
                               const int64_t* idx, const float* q1, const float* q2, const float* score,
                               const float* gscore, float* gq1, float* gq2, size_t B, size_t K, size_t dim,
                               const smx_score_params* params, float* merged, float* m, float* v,
                               const smx_opt_params* adam, void* workspace, size_t workspace_bytes,
                               const void* fwd_codes, size_t fwd_codes_bytes) {
  if (parts < 1 || parts > 3) return smx::fail(SMX_ERR_ARG, "backward parts must be 1, 2 or 3");
  return smx::backward_fused(parts, model, stream, plan, table, n_rows, idx, q1, q2, score, gscore, gq1, gq2, B, K, dim,
                             params, merged, m, v, adam, workspace, workspace_bytes, fwd_codes, fwd_codes_bytes);
}

}  // extern "C"
