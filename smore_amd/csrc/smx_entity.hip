// Entity-side backward: segmented gradient reduction with the sparse Adam row
// update fused into the same pass.  No float atomics anywhere; every sum has a
// fixed order, so two runs on the same inputs give the same bits.
//
// Replaces, per training step,
//   dist_backward_ent_kernel              smore/common/torchext/common_kernel.h:59-89
//   EmbedLookupFunc.backward / accumulate smore/common/embedding/embed_optimizer.py:63-66,146-148
//   merge_grad_list (scatter-sum)         embed_optimizer.py:45-48
//   AdamEmbedOptimizer.update_step        embed_optimizer.py:208-252
// The reference materialises a [P, row] gradient tensor, scatter-adds it into
// [U, row] and then runs ~20 row-sized tensor passes for Adam.  Here the sorted
// pair list of the segment plan is cut into fixed tiles; one wavefront walks a
// tile, recomputes each pair's entity gradient from (entity row, query row,
// upstream gradient) in registers -- or, for gradients that autograd already
// materialised, reads the pair's gradient row -- and sums it per segment.
//   * a segment that lies inside one tile is finished on the spot: the lanes
//     holding its gradient read w, m, v of that entity row, apply Adam, and
//     write the three rows back;
//   * a segment crossing a tile edge leaves one partial row per tile (tail: it
//     continues past the tile end; head: it came in from the left and ends
//     here); a second kernel adds the partials of such a segment in tile order
//     and then finishes it the same way.
// Consecutive pairs of a segment that belong to the same query (common when
// ids repeat inside one query's negatives) share one gradient evaluation: the
// derivative is linear in the upstream coefficient, so coefficients are summed
// first.
#include <cmath>

#include "smx_entity_impl.h"

namespace smx {

extern template int entity_dispatch<mL1>(hipStream_t, const EntityArgs&, int, int);
extern template int entity_dispatch<mL2>(hipStream_t, const EntityArgs&, int, int);
extern template int entity_dispatch<mBox>(hipStream_t, const EntityArgs&, int, int);
extern template int entity_dispatch<mRotate>(hipStream_t, const EntityArgs&, int, int);
extern template int entity_dispatch<mBetaKL>(hipStream_t, const EntityArgs&, int, int);
extern template int entity_dispatch<mComplex>(hipStream_t, const EntityArgs&, int, int);
extern template int entity_dispatch<mDistmult>(hipStream_t, const EntityArgs&, int, int);
extern template int entity_dispatch<kSrcRows>(hipStream_t, const EntityArgs&, int, int);

static size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

struct EntityScratch {
  size_t tail_off, head_off, fix_off, total;
};
constexpr size_t kFixHeader = 64;  // ints in front of the fix-up list; the first is the list's length

static EntityScratch entity_scratch(size_t n_pairs, size_t row_len) {
  const size_t tiles = (n_pairs + kTile - 1) / kTile;
  EntityScratch s;
  s.tail_off = 0;
  s.head_off = align256(tiles * row_len * sizeof(float));
  s.fix_off = s.head_off + align256(tiles * row_len * sizeof(float));
  s.total = s.fix_off + align256((tiles + kFixHeader) * sizeof(int));
  return s;
}

size_t entity_ws_bytes(size_t n_pairs, size_t row_len) { return entity_scratch(n_pairs, row_len).total; }

// Sign codes: one byte per lane and column group of 64 lanes; the groups are those of the float4 layout
// when dim allows it (rows that are then not 16-byte aligned get no codes), of single floats otherwise.
size_t code_bytes_per_pair(size_t dim) {
  const size_t ncol = dim % 4 == 0 ? dim / 4 : dim;
  size_t groups = (ncol + 63) / 64, g = 1;
  while (g < groups) g *= 2;
  return g * 64;
}

static int fill_plan(EntityArgs* A, const smx_plan_view* plan, void* workspace, size_t workspace_bytes, size_t row_len) {
  if (!plan || !plan->order || !plan->sorted_ids || !plan->seg_of_pos || !plan->seg_start || !plan->uniq ||
      !plan->n_uniq)
    return fail(SMX_ERR_ARG, "incomplete segment plan");
  if (plan->n_pairs == 0 || plan->n_pairs > 0x7fffffffull) return fail(SMX_ERR_SHAPE, "pair count out of range");
  const EntityScratch sc = entity_scratch(plan->n_pairs, row_len);
  if (!workspace || workspace_bytes < sc.total)
    return fail(SMX_ERR_WORKSPACE, "entity workspace too small: %zu < %zu", workspace_bytes, sc.total);
  if (reinterpret_cast<uintptr_t>(workspace) & 255u) return fail(SMX_ERR_ARG, "workspace must be 256-byte aligned");
  A->order = plan->order;
  A->sorted_ids = plan->sorted_ids;
  A->seg_of_pos = plan->seg_of_pos;
  A->seg_start = plan->seg_start;
  A->uniq = reinterpret_cast<const long long*>(plan->uniq);
  A->n_uniq = plan->n_uniq;
  A->n_pairs = (int)plan->n_pairs;
  A->rows_first = (int)plan->n_pairs;  // no gradient rows of plain lookups behind the model's pairs
  A->tile = kTile;
  A->short_max = kShortMax;
  A->chunk = 64;  // enough wavefronts to fill the chip also for a short list
  while (A->chunk > 1 && plan->n_pairs / (size_t)A->chunk < 4096) A->chunk /= 2;
  char* ws = static_cast<char*>(workspace);
  A->tail = reinterpret_cast<float*>(ws + sc.tail_off);
  A->head = reinterpret_cast<float*>(ws + sc.head_off);
  A->fix_count = reinterpret_cast<int*>(ws + sc.fix_off);
  A->fix_list = A->fix_count + kFixHeader;
  return SMX_OK;
}

int entity_backward(int model, void* stream, const smx_plan_view* plan, float* table, size_t n_rows, const float* q1,
                    const float* q2, const float* score, const float* gscore, size_t B, size_t K, size_t dim,
                    const smx_score_params* params, float* merged, float* m, float* v, const smx_opt_params* adam,
                    void* workspace, size_t workspace_bytes, int skip_single, const unsigned char* codes, int codes_vec,
                    int codes_nit, const PairSources* multi = nullptr);

static int fill_adam(EntityArgs* A, float* m, float* v, const smx_opt_params* opt) {
  A->adam_on = 0;
  A->squeeze = 0;
  A->m = m;
  A->v = v;
  if (opt) {
    if (const char* msg = check_opt_params(opt, m, v)) return fail(SMX_ERR_ARG, "%s", msg);
    A->adam_on = opt->kind;
    A->squeeze = opt->squeeze ? 1 : 0;
    A->a = make_adam_consts(opt);
    A->step_dev = opt->step_consts_dev;
  } else if (m || v) {
    return fail(SMX_ERR_ARG, "optimizer state given without optimizer parameters");
  }
  return SMX_OK;
}

}  // namespace smx

extern "C" {

size_t smx_entity_workspace_bytes(size_t n_pairs, size_t row_len) { return smx::entity_ws_bytes(n_pairs, row_len); }

int smx_opt_step_consts(const smx_opt_params* opt, float* out2) {
  using namespace smx;
  if (!opt || !out2) return fail(SMX_ERR_ARG, "null pointer");
  if (opt->kind < SMX_OPT_ADAM || opt->kind > SMX_OPT_RMSPROP) return fail(SMX_ERR_ARG, "unknown optimizer kind");
  if (opt->kind == SMX_OPT_ADAM && opt->step < 1) return fail(SMX_ERR_ARG, "Adam step counter starts at 1");
  step_consts(opt, out2);
  return SMX_OK;
}

size_t smx_fused_workspace_bytes(int model, size_t n_pairs, size_t dim) {
  using namespace smx;
  if (model < 0 || model >= mNumModels) return 0;
  size_t total = entity_ws_bytes(n_pairs, dim * model_mul(model));
  if (model_coded(model)) total += align256(n_pairs * code_bytes_per_pair(dim));
  return total;
}

}  // extern "C"

namespace smx {

int entity_backward(int model, void* stream, const smx_plan_view* plan, float* table, size_t n_rows, const float* q1,
                    const float* q2, const float* score, const float* gscore, size_t B, size_t K, size_t dim,
                    const smx_score_params* params, float* merged, float* m, float* v, const smx_opt_params* adam,
                    void* workspace, size_t workspace_bytes, int skip_single, const unsigned char* codes, int codes_vec,
                    int codes_nit, const PairSources* multi) {
  if (model < 0 || model >= mNumModels) return fail(SMX_ERR_KIND, "unknown score model %d", model);
  if (!table || !q1 || (!multi && (!score || !gscore)) || !params || (model_nq(model) == 2 && !q2))
    return fail(SMX_ERR_ARG, "null pointer");
  if (B == 0 || K == 0 || dim == 0 || n_rows == 0) return fail(SMX_ERR_SHAPE, "empty dimension");
  if (const char* why = params_refused(model, params)) return fail(SMX_ERR_ARG, "%s", why);
  if (!merged && !adam) return fail(SMX_ERR_ARG, "nothing to do: neither merged gradient nor an optimizer requested");
  EntityArgs A{};
  const size_t row_len = dim * model_mul(model);
  if (int rc = fill_plan(&A, plan, workspace, workspace_bytes, row_len)) return rc;
  const size_t n_grad = multi ? multi->n_grad : 0;
  // the model's pairs: B * K, or what the sources hold (a source has its own K and, when the sources belong to
  // different query batches, its own stretch of the B query rows)
  size_t n_model = B * K;
  if (multi) {
    if (multi->n < 1 || multi->n > kMaxSources) return fail(SMX_ERR_ARG, "1 to %d pair sources", kMaxSources);
    A.n_src = multi->n;
    size_t first = 0;
    for (int i = 0; i < multi->n; ++i) {
      if (!multi->score[i] || !multi->gscore[i] || multi->K[i] == 0) return fail(SMX_ERR_ARG, "incomplete pair source %d", i);
      if ((codes != nullptr) != (multi->codes[i] != nullptr)) return fail(SMX_ERR_ARG, "sign codes for some pair sources only");
      if (multi->B[i] == 0 || multi->q_first[i] + multi->B[i] > B)
        return fail(SMX_ERR_SHAPE, "pair source %d: queries %zu .. %zu of %zu", i, multi->q_first[i],
                    multi->q_first[i] + multi->B[i], B);
      A.first[i] = (int)first;
      A.src_score[i] = multi->score[i];
      A.src_gscore[i] = multi->gscore[i];
      A.src_codes[i] = multi->codes[i];
      A.src_K[i] = (int)multi->K[i];
      A.src_q0[i] = (int)multi->q_first[i];
      A.src_winner[i] = multi->winner[i];
      first += multi->B[i] * multi->K[i];
    }
    for (int i = multi->n; i <= kMaxSources; ++i) A.first[i] = (int)first;
    n_model = first;
  }
  if (plan->n_pairs != n_model + n_grad)
    return fail(SMX_ERR_SHAPE, "plan holds %zu pairs, call has %zu", plan->n_pairs, n_model + n_grad);
  if (n_grad) {
    if (!multi->grad_rows) return fail(SMX_ERR_ARG, "null gradient rows");
    A.grad_rows = multi->grad_rows;
    A.rows_first = (int)n_model;
  }
  if (int rc = fill_adam(&A, m, v, adam)) return rc;
  const bool vec4 = dim % 4 == 0 && aligned16(table) && aligned16(q1) && (!q2 || aligned16(q2)) &&
                    (!merged || aligned16(merged)) && (!m || aligned16(m)) && (!v || (adam && adam->squeeze) || aligned16(v)) &&
                    (!n_grad || aligned16(multi->grad_rows));
  const int vec = vec4 ? 4 : 1;
  const size_t ncol = dim / vec;
  if (ncol > 512) return fail(SMX_ERR_SHAPE, "dim %zu not supported by the fused path", dim);
  const int need = (int)((ncol + 63) / 64);
  const int nit = need <= 1 ? 1 : (need <= 2 ? 2 : (need <= 4 ? 4 : 8));
  if (vec == 1 && nit > 4) return fail(SMX_ERR_SHAPE, "rows of %zu unaligned floats are not supported by the fused path", (size_t)ncol);
  A.q1 = q1;
  A.q2 = q2;
  A.score = score;
  A.gscore = gscore;
  A.K = (int)K;
  A.U = 1;
  if (multi && multi->U > 1) {
    if (codes) return fail(SMX_ERR_ARG, "union queries have no sign codes");
    for (int i = 0; i < multi->n; ++i)
      if (!multi->winner[i]) return fail(SMX_ERR_ARG, "union queries: pair source %d has no winner array", i);
    A.U = (int)multi->U;
  }
  if (multi && multi->n == 1) {  // one index stream (+ gradient rows): the single-source fields describe it
    if (multi->q_first[0] != 0) return fail(SMX_ERR_ARG, "a single pair source starts at the first query");
    A.n_src = 0;
    A.score = multi->score[0];
    A.gscore = multi->gscore[0];
    A.winner = multi->winner[0];
  }
  A.p = to_params(params);
  A.table = table;
  A.merged = merged;
  A.ncol = (int)ncol;
  A.skip_single = skip_single;
  if (codes) {
    if (vec != codes_vec || nit != codes_nit) return fail(SMX_ERR_ARG, "sign codes were written for another column layout");
    A.codes = codes;
  }
  hipStream_t st = as_stream(stream);
  switch (model) {
    case mL1: return entity_dispatch<mL1>(st, A, vec, nit);
    case mL2: return entity_dispatch<mL2>(st, A, vec, nit);
    case mBox: return entity_dispatch<mBox>(st, A, vec, nit);
    case mRotate: return entity_dispatch<mRotate>(st, A, vec, nit);
    case mBetaKL: return entity_dispatch<mBetaKL>(st, A, vec, nit);
    case mComplex: return entity_dispatch<mComplex>(st, A, vec, nit);
    case mDistmult: return entity_dispatch<mDistmult>(st, A, vec, nit);
  }
  return fail(SMX_ERR_KIND, "unknown score model %d", model);
}

}  // namespace smx

extern "C" {

int smx_rows_backward(void* stream, const smx_plan_view* plan, const float* grad_rows, size_t row_len, float* merged,
                      float* table, float* m, float* v, const smx_opt_params* adam, void* workspace,
                      size_t workspace_bytes) {
  using namespace smx;
  if (!grad_rows || row_len == 0) return fail(SMX_ERR_ARG, "null gradient rows");
  if (!merged && !adam) return fail(SMX_ERR_ARG, "nothing to do: neither merged gradient nor an optimizer requested");
  EntityArgs A{};
  if (int rc = fill_plan(&A, plan, workspace, workspace_bytes, row_len)) return rc;
  if (int rc = fill_adam(&A, m, v, adam)) return rc;
  if (A.adam_on && !table) return fail(SMX_ERR_ARG, "Adam needs the weight table");
  const bool vec4 = row_len % 4 == 0 && aligned16(grad_rows) && (!merged || aligned16(merged)) &&
                    (!A.adam_on || (aligned16(table) && (!m || aligned16(m)) && (!v || A.squeeze || aligned16(v))));
  const int vec = vec4 ? 4 : 1;
  const size_t ncol = row_len / vec;
  if (ncol > 512) return fail(SMX_ERR_SHAPE, "row length %zu not supported by the fused path", row_len);
  const int need = (int)((ncol + 63) / 64);
  const int nit = need <= 1 ? 1 : (need <= 2 ? 2 : (need <= 4 ? 4 : 8));
  if (vec == 1 && nit > 4) return fail(SMX_ERR_SHAPE, "rows of %zu unaligned floats are not supported by the fused path", (size_t)ncol);
  A.grad_rows = grad_rows;
  A.table = table;
  A.merged = merged;
  A.ncol = (int)ncol;
  A.K = 1;
  return entity_dispatch<kSrcRows>(as_stream(stream), A, vec, nit);
}

}  // extern "C"
