/*
 * smore_amd -- C ABI of the MI355X (gfx950) scoring path for SMORE.
 *
 * The library replaces the native waist of SMORE's `extlib_cuda` distance
 * operators and the tensor pipeline of its sparse row optimizer.  Every entry
 * point takes plain device pointers and sizes, launches asynchronously on the
 * HIP stream it is given (NULL = the default stream), allocates nothing on the
 * device and returns a status code; smx_last_error() gives the text of the
 * last failure on the calling thread.  Citations name the reference interface
 * (paths relative to the SMORE checkout) each function stands in for.
 *
 * Layout: all tensors are contiguous row-major, last dimension fastest.
 * Entity rows are `dim * mul` long, mul = 2 for the kinds whose row is two
 * halves [first | second] (rotate, complex, beta_*), else 1.
 */
#ifndef SMORE_AMD_H
#define SMORE_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* status codes */
#define SMX_OK 0
#define SMX_ERR_KIND 1      /* unknown operator kind / model */
#define SMX_ERR_SHAPE 2     /* sizes do not fit the operator's contract */
#define SMX_ERR_ARG 3       /* null or misaligned pointer */
#define SMX_ERR_HIP 4       /* the HIP runtime reported an error at launch */
#define SMX_ERR_WORKSPACE 5 /* workspace too small */

/* operator kinds: the dist_name strings of smore/common/torchext/ext_cuda_kernel.cu:25-49 */
#define SMX_KIND_L1 0          /* "l1" */
#define SMX_KIND_L2 1          /* "l2" (squared distance) */
#define SMX_KIND_BOX_OUT 2     /* "box_out" */
#define SMX_KIND_BOX_IN 3      /* "box_in" */
#define SMX_KIND_ROTATE 4      /* "rotate" */
#define SMX_KIND_BETA_KL 5     /* "beta_kl" */
#define SMX_KIND_COMPLEX 6     /* "complex" */
#define SMX_KIND_DISTMULT 7    /* "distmult" */
#define SMX_KIND_BETA_L2 8     /* "beta_l2" */
#define SMX_KIND_BETA_FISHER 9 /* "beta_fisher_approx" */

/* score models of the fused path: the custom_cal_logit bodies of smore/models */
#define SMX_MODEL_L1 0      /* gamma - sum|e-q|                    models/vec.py:85-90 */
#define SMX_MODEL_L2 1      /* gamma - sqrt(sum (e-q)^2)           torchext/dist_func/l2_dist.py:59-62 */
#define SMX_MODEL_BOX 2     /* gamma - d_out - cen * d_in          models/box.py:157-164 */
#define SMX_MODEL_ROTATE 3  /* gamma - sum sqrt(dre^2 + dim^2)     models/rotate.py:137-142 */
#define SMX_MODEL_BETA_KL 4 /* gamma - sum KL(Beta(e) || Beta(q))  models/beta.py:303-308 */
#define SMX_MODEL_COMPLEX 5 /* gamma + sum (e_re q_re + e_im q_im)  models/complex.py:140-148 (gamma = 0 there) */
#define SMX_MODEL_DISTMULT 6 /* gamma + sum e q                     models/distmult.py, distmult_sim (gamma = 0 there) */

int smx_version(void);
const char* smx_last_error(void);

/* Process-wide switches (thread-safe; take effect for calls made afterwards).  None changes a result.
 *   SMX_OPTION_SERIAL_BACKWARD  != 0: smx_score_backward_fused / smx_score_backward_entity keep all their
 *                               kernels on the caller's stream instead of running the entity pass on the
 *                               library's second stream -- same results, for per-kernel profiling. */
#define SMX_OPTION_SERIAL_BACKWARD 1
int smx_set_option(int option, int value);

/* kind id for a dist_name string ("l1", "box_out", ...), -1 if unknown.
 * Replaces the string chain of ext_cuda_kernel.cu:25-49 (which prints and
 * silently does nothing for an unknown name; here the caller gets -1). */
int smx_kind_from_name(const char* dist_name);

/* ---- dense operators ------------------------------------------------------
 * Replace DistImpl<scalar_t>::forward / ::backward
 * (smore/common/torchext/ext_cuda_kernel.h:29-30, reached from
 * extlib_cuda.cpp:172-196 and :230-262).
 *   ent  [be, ne, dim*mul]   q1, q2 [bc, nc, dim]   dst / gout [bsize, num]
 *   dst[i,j] = sum_d f(ent[i%be, j%ne], q[i%bc, j%nc], d)
 * q2 (and gq2) are NULL for the one-query kinds, as has_second=false passes
 * nullptr there.  backward overwrites gent, gq1, gq2 (no zero-fill needed). */
int smx_dist_forward_f32(int kind, void* stream, const float* ent, const float* q1, const float* q2,
                         float* dst, size_t bsize, size_t num, size_t be, size_t ne, size_t bc,
                         size_t nc, size_t dim);
int smx_dist_forward_f64(int kind, void* stream, const double* ent, const double* q1,
                         const double* q2, double* dst, size_t bsize, size_t num, size_t be,
                         size_t ne, size_t bc, size_t nc, size_t dim);
int smx_dist_backward_f32(int kind, void* stream, const float* gout, const float* ent,
                          const float* q1, const float* q2, float* gent, float* gq1, float* gq2,
                          size_t bsize, size_t num, size_t be, size_t ne, size_t bc, size_t nc,
                          size_t dim);
int smx_dist_backward_f64(int kind, void* stream, const double* gout, const double* ent,
                          const double* q1, const double* q2, double* gent, double* gq1,
                          double* gq2, size_t bsize, size_t num, size_t be, size_t ne, size_t bc,
                          size_t nc, size_t dim);

/* ---- gather-fused scoring -------------------------------------------------
 * One training step scores every (query b, negative k) pair against the entity
 * row table[idx[b,k]].  These entry points fuse what the reference runs as
 * separate steps, without materialising the gathered [B,K,row] tensor:
 *   rows = table[idx]            smore/common/embedding/embed_rw.py:74-75
 *                                (EmbedLookupFunc.forward, embed_optimizer.py:51-61)
 *   clamp(rows + add, lo, hi)    smore/common/modules.py:29-36 (BetaE only)
 *   dist forward / backward      smore/common/torchext/common_kernel.h:33-123
 *   logit = gamma - dist         custom_cal_logit of smore/models/{vec,box,rotate,beta}.py
 *   table [n_rows, dim*mul] fp32   idx [B,K] int64   q1, q2 [B, dim]   score [B,K]
 * idx == NULL means `table` already holds the B*K rows in pair order (the
 * dense [B,K,row] layout of the reference operators).
 * An id outside [0, n_rows) sets *err_flag (device int, may be NULL) to 1 and
 * row 0 is read in its place for the score and the query gradient; the caller
 * decides when to look at the flag.  No table row is ever updated for such a
 * pair (see smx_plan_build).  With an id list, n_rows is at most 2^32 - 1
 * (SMX_ERR_SHAPE beyond: ids are told apart by their low 32 bits, as in the
 * segment plan). */
typedef struct smx_score_params {
  float gamma;   /* margin: logit = gamma - distance */
  float cen;     /* BOX: weight of the inside distance */
  int reg_on;    /* apply clamp(e + reg_add, reg_lo, reg_hi) to entity values */
  float reg_add;
  float reg_lo;
  float reg_hi;
  int norm_on;   /* COMPLEX: each half of an entity row (re, im) is scaled to unit L2 length before it is scored
                  * (complex.py:142-146 with the 'norm' mode of complex.py:87-89: F.normalize, eps 1e-12), and the
                  * entity gradient is taken through that scaling.  DISTMULT: the same with the whole row
                  * (distmult.py:85-87,129-130).  Other models refuse it (SMX_ERR_ARG). */
} smx_score_params;

/* Sign codes (optional, what autograd would call a saved tensor).  For the box model (and, with one
 * decision per feature, L1) the derivative
 * of a pair's distance w.r.t. each feature is +-c0 or +-c1, decided by comparisons the forward pass
 * makes anyway.  Given a `codes` buffer of smx_score_codes_bytes(model, B*K, dim) bytes (16-byte
 * aligned), the forward leaves those decisions there, two bits per feature; handed to
 * smx_score_backward_fused, they replace every read of entity and query rows for the gradient -- the
 * same decisions, hence the same bits as recomputing them, as long as table and queries are unchanged
 * between the two calls.  smx_score_codes_bytes is 0 for models or row lengths without codes (pass
 * codes = NULL then). */
size_t smx_score_codes_bytes(int model, size_t n_pairs, size_t dim);

int smx_score_forward(int model, void* stream, const float* table, size_t n_rows, const int64_t* idx,
                      const float* q1, const float* q2, float* score, size_t B, size_t K, size_t dim,
                      const smx_score_params* params, int* err_flag, void* codes, size_t codes_bytes);

/* Query-side gradient of sum(gscore * score): gq1, gq2 [B, dim] are overwritten.
 * `score` is the tensor smx_score_forward wrote (L2 needs it for the chain
 * rule of the square root).  Replaces dist_backward_query_kernel
 * (common_kernel.h:92-123) plus the autograd nodes between it and the logit.
 * fwd_codes (may be NULL): the sign codes smx_score_forward wrote for these pairs; the kernel then
 * reads them instead of the entity rows. */
int smx_score_backward_query(int model, void* stream, const float* table, size_t n_rows,
                             const int64_t* idx, const float* q1, const float* q2,
                             const float* score, const float* gscore, float* gq1, float* gq2,
                             size_t B, size_t K, size_t dim, const smx_score_params* params,
                             const void* fwd_codes, size_t fwd_codes_bytes);

/* ---- segment plan ----------------------------------------------------------
 * Groups the P = B*K pairs of a step by entity id on the device.  Replaces
 * merge_grad_indices (smore/common/embedding/embed_optimizer.py:39-42), i.e.
 * torch.unique(ids, return_inverse=True) run on the host.  Integer outputs are
 * bit-exact by contract:
 *   order[P]       pair positions grouped by id; inside an id ascending (stable)
 *   sorted_ids[P]  idx[order[.]] as 32-bit ids (read as unsigned)
 *   seg_of_pos[P]  segment number of every sorted position
 *   uniq[P]        first n_uniq entries: the distinct ids, ascending (= torch.unique)
 *   seg_start[P+1] first n_uniq+1 entries: start of each segment in order[]
 *   inverse[P]     position of idx[p] in uniq (= return_inverse), may be NULL
 *   pair_seg[P]    per pair: sign bit + segment number when the pair is alone in its segment (its
 *                  id occurs once in the step), 0 otherwise; may be NULL
 *   n_uniq         device int: number of distinct ids
 * All arrays are caller-allocated device memory.  workspace: at least
 * smx_plan_workspace_bytes(P, n_rows) bytes (ask with the device current that the build will run on),
 * 256-byte aligned.  Needs n_rows < 2^32.
 * The build is kernel launches only (an LSD radix sort written for this shape, then one pass that numbers
 * the segments): no library call, no memset, so it can be recorded into a HIP graph with the rest of a step.
 * Ids outside [0, n_rows) set *err_flag = 1 and sort behind every valid id as one last segment that is not
 * counted in n_uniq, is skipped by the entity pass and is never a one-pair segment: no row is updated for
 * them (inverse[] holds n_uniq for such pairs).  *err_flag = 2: a workgroup of the sort gave up waiting for
 * another one (bounded wait, never seen in practice); *n_uniq is then -1, and every entry point that is handed
 * such a plan does nothing (its kernels look at n_uniq before anything else of the plan).
 * Up to 4096 ids are sorted by one workgroup in one launch (the ids of a step whose negatives are shared by the
 * batch: K + B + anchors); the workspace is not used then. */
size_t smx_plan_workspace_bytes(size_t n_pairs, size_t n_rows);
int smx_plan_build(void* stream, const int64_t* idx, size_t n_pairs, size_t n_rows, void* workspace,
                   size_t workspace_bytes, int32_t* order, int32_t* sorted_ids, int32_t* seg_of_pos,
                   int64_t* uniq, int32_t* seg_start, int64_t* inverse, int32_t* pair_seg,
                   int32_t* n_uniq, int* err_flag);

typedef struct smx_plan_view {
  const int32_t* order;
  const int32_t* sorted_ids;
  const int32_t* seg_of_pos;
  const int32_t* seg_start;
  const int64_t* uniq;
  const int32_t* n_uniq;   /* device scalar */
  const int32_t* pair_seg; /* may be NULL where the one-pair fast path is not used */
  size_t n_pairs;
} smx_plan_view;

/* Row optimizers of smore/common/embedding/embed_optimizer.py, all lazy (touched rows only):
 *   ADAM    AdamEmbedOptimizer.update_step :208-252 (global step counter, eps = common/consts.py:20)
 *   SGD     SGDEmbedOptimizer.update_step :174-178
 *   ADAGRAD AdaGradEmbedOptimizer.update_step :327-349
 *   RMSPROP RMSpropEmbedOptimizer.update_step :271-309 (its alpha = 0.99 goes in beta2)
 * `step` is the counter after apply_grad incremented it (:156): the first update has step = 1.
 * squeeze != 0: the second-moment state v is one float per row ([N] / [N,1]) fed by the row mean of
 * g*g (optim_mode[3] of the reference, :220-221, :237-238, :336-337).  State tables: ADAM uses m and v,
 * ADAGRAD / RMSPROP use v only (m may be NULL), SGD none. */
#define SMX_OPT_ADAM 1
#define SMX_OPT_SGD 2
#define SMX_OPT_ADAGRAD 3
#define SMX_OPT_RMSPROP 4
typedef struct smx_opt_params {
  double lr;    /* hyper-parameters are doubles, as the Python floats of the reference are: */
  double beta1; /* 1 - beta is formed in double and only then rounded to fp32             */
  double beta2;
  double eps;
  long step;
  int kind;     /* SMX_OPT_* */
  int squeeze;
  /* NULL, or device memory with the two per-step constants smx_opt_step_consts() computes; the kernels
   * then read them at run time instead of taking them from lr / step above.  A launch recorded into a
   * HIP graph freezes its arguments: with this buffer (rewritten by the caller between replays) a
   * captured step follows the learning-rate schedule and Adam's bias correction; without it every
   * replay repeats the lr and step of the capture. */
  const float* step_consts_dev;
} smx_opt_params;

/* out2[0] = -lr / (1 - beta1^step), out2[1] = 1 / sqrt(1 - beta2^step) for ADAM (embed_optimizer.py:241-249),
 * { -lr, 1 } for the other kinds: the contents of smx_opt_params.step_consts_dev.  Host-only. */
int smx_opt_step_consts(const smx_opt_params* opt, float* out2);

/* ---- entity-side backward, segment sum and row update in one pass ----------
 * For every distinct id u of the plan: g[u,:] = sum over the pairs of segment u
 * of d(sum gscore*score)/d(entity row), summed in the plan's order (fixed, no
 * atomics).  Then, as requested:
 *   merged != NULL   merged[u,:] = g[u,:]        ([n_uniq, dim*mul], caller-sized for P rows
 *                                                 or fewer if it knows n_uniq)
 *   adam given       table[id] and the optimizer's state rows m[id], v[id] are updated in place
 *                    (see smx_opt_params for which state a kind uses); rows of ids not in the
 *                    plan are not touched.
 * Replaces dist_backward_ent_kernel (common_kernel.h:59-89), EmbedLookupFunc.backward
 * (embed_optimizer.py:63-66), merge_grad_list (:45-48) and update_step (:208-252).
 * workspace: smx_entity_workspace_bytes(P, dim*mul) bytes, 256-byte aligned.
 * fwd_codes (may be NULL): the forward's sign codes; they replace the reads of the query rows.
 * With them, an optimizer, no merged output and a step of a million pairs or more whose queries
 * exceed one L2, the call finishes ids that occur once in a pair-ordered kernel on `stream` and
 * reduces the others on the library's second stream beside it (joined to `stream` before return);
 * the rows get the same bits either way (smx_set_option(SMX_OPTION_SERIAL_BACKWARD, 1) keeps this call
 * and smx_score_backward_fused on the caller's stream alone). */
size_t smx_entity_workspace_bytes(size_t n_pairs, size_t row_len);
int smx_score_backward_entity(int model, void* stream, const smx_plan_view* plan, float* table,
                              size_t n_rows, const float* q1, const float* q2, const float* score,
                              const float* gscore, size_t B, size_t K, size_t dim,
                              const smx_score_params* params, float* merged, float* m, float* v,
                              const smx_opt_params* adam, void* workspace, size_t workspace_bytes,
                              const void* fwd_codes, size_t fwd_codes_bytes);

/* The same pass over several index streams that share one query batch -- a step's positives [B,1] and
 * negatives [B,K] scored against the same query embeddings (kg_reasoning.py:340-355), each by its own
 * smx_score_forward call.  Replaces what the reference does with several (indices, gradient rows) records in
 * apply_grad (embed_optimizer.py:155-163): concatenate, merge_grad_indices (:39-42), merge_grad_list (:45-48),
 * one update_step per entity (:208-252) -- without materialising gradient rows.
 * plan: built by smx_plan_build over the concatenation [ids of source 0 (B*K_0) | ids of source 1 (B*K_1) | ..];
 * pair j of source s (query j / K_s) is pair B*(K_0 + .. + K_s-1) + j of the plan.  Every source brings the
 * score its forward produced, the upstream gradient, and its sign codes (all sources or none); q1, q2, B, dim,
 * params are common to all.  An entity that occurs in several sources gets ONE update from the sum of all its
 * pairs' gradients, summed in plan order (source by source, pairs ascending).  n_src == 1 is
 * smx_score_backward_entity.
 * grad_rows (may be NULL): [n_grad_rows, dim*mul] gradient rows that autograd has materialised for the step's
 * plain lookups -- the anchor entities every query starts from (models/box.py:137), which reach the optimizer
 * as (indices, gradient rows) records of their own (embed_optimizer.py:63-66, 146-148).  Their ids are the last
 * n_grad_rows entries of the plan's concatenation; a row is added to its entity's gradient after the model's own
 * part is complete (clamp mask of the entity prologue included), so that such an entity too gets ONE update.
 * workspace: smx_entity_workspace_bytes(plan->n_pairs, dim*mul). */
#define SMX_MAX_PAIR_SOURCES 4
typedef struct smx_pair_source {
  const float* score;      /* [B, K] */
  const float* gscore;     /* [B, K] */
  const void* fwd_codes;   /* may be NULL */
  size_t fwd_codes_bytes;
  size_t K;
  const uint8_t* winner;   /* [B, K] union queries only (smx_score_backward_entity_union), else NULL */
  size_t q_first;          /* first query (row of q1 / q2; with union queries: group of U rows) of this source */
  size_t n_queries;        /* queries of this source; 0 = B, all of them */
} smx_pair_source;
int smx_score_backward_entity_multi(int model, void* stream, const smx_plan_view* plan, float* table,
                                    size_t n_rows, const float* q1, const float* q2,
                                    const smx_pair_source* src, size_t n_src, size_t B, size_t dim,
                                    const smx_score_params* params, float* merged, float* m, float* v,
                                    const smx_opt_params* adam, void* workspace, size_t workspace_bytes,
                                    const float* grad_rows, size_t n_grad_rows);

/* ---- union queries ---------------------------------------------------------------------------
 * A query in disjunctive normal form has U branch embeddings (smore/models/kg_reasoning.py:326), and the last line
 * of every custom_cal_logit takes the maximum of the branches' logits (box.py:163, vec.py:89, rotate.py:141,
 * beta.py:307).  q1, q2 are [B, U, dim] (branch rows of one query adjacent), idx [B, K] as for one branch.
 *   smx_score_forward_union         score[b,k] = max_u logit(table[idx[b,k]], q[b,u]); winner[b,k] = the first
 *                                   branch that holds the maximum (values / indices of torch.max(logit, dim=1)).
 *                                   workspace: smx_union_workspace_bytes(B, U, K), every branch's logits.
 *   smx_score_backward_query_union  gq1, gq2 [B, U, dim]: a branch row gets the gradient of the pairs it won
 *                                   (autograd of torch.max), summed in pair order; it streams those pairs only.
 *   smx_score_backward_entity_union smx_score_backward_entity_multi for such queries: every source brings its
 *                                   winner array, a pair's entity gradient is taken against the branch that won
 *                                   it, and the plan is built over the B*K pairs of each source, not over B*U*K.
 *                                   No sign codes with union queries (pass fwd_codes = NULL).
 * Replaces the same reference functions as the one-branch entry points, plus torch.max and its backward. */
size_t smx_union_workspace_bytes(size_t B, size_t U, size_t K);
int smx_score_forward_union(int model, void* stream, const float* table, size_t n_rows, const int64_t* idx,
                            const float* q1, const float* q2, float* score, uint8_t* winner, size_t B, size_t U,
                            size_t K, size_t dim, const smx_score_params* params, int* err_flag, void* workspace,
                            size_t workspace_bytes);
int smx_score_backward_query_union(int model, void* stream, const float* table, size_t n_rows, const int64_t* idx,
                                   const float* q1, const float* q2, const float* score, const float* gscore,
                                   const uint8_t* winner, float* gq1, float* gq2, size_t B, size_t U, size_t K,
                                   size_t dim, const smx_score_params* params);
int smx_score_backward_entity_union(int model, void* stream, const smx_plan_view* plan, float* table,
                                    size_t n_rows, const float* q1, const float* q2, const smx_pair_source* src,
                                    size_t n_src, size_t B, size_t U, size_t dim, const smx_score_params* params,
                                    float* merged, float* m, float* v, const smx_opt_params* adam, void* workspace,
                                    size_t workspace_bytes, const float* grad_rows, size_t n_grad_rows);

/* Everything after the loss in one call: query gradients, and every entity row of the step finished
 * (merged gradient row and/or lazy Adam on w, m, v), as smx_score_backward_query followed by
 * smx_score_backward_entity would do -- except that rows of ids occurring once in the step are
 * finished by the query-gradient kernel itself, which already holds the query in registers and has
 * just read the entity row; the entity pass then skips them.  The plan must have been built with
 * pair_seg.  Against the two separate calls: query gradients and the w, m, v rows of the sign-coded models
 * (box, l1) are the same bits -- same decisions, same +-c terms, same order, and the row update is written
 * with explicit fused multiply-adds, so it does not depend on the kernel that runs it.  For l2, rotate and
 * beta_kl the gradient of a one-pair row is formed by the query-gradient kernel instead of the entity pass,
 * whose multiply-adds the compiler contracts differently: merged gradient rows agree to a few units of the
 * last place (the tests bound the difference by 1e-6 relative).
 * workspace: smx_fused_workspace_bytes (below).  No counterpart as one function in the reference:
 * it stands for dist_backward (extlib_cuda.cpp:230-262) + EmbedLookupFunc.backward +
 * EmbeddingOptimizer.apply_grad (embed_optimizer.py:63-66,155-163). */
/* Workspace of smx_score_backward_fused: smx_entity_workspace_bytes(P, dim*mul) plus, for models whose
 * entity derivative is a choice of sign and coefficient (box), room for the per-pair sign codes the
 * query-gradient kernel leaves for the entity pass (64 bytes per pair and 256 floats of dim).  With
 * only smx_entity_workspace_bytes the call works too and the entity pass reads the query rows.
 * fwd_codes (may be NULL): the codes smx_score_forward wrote for these same pairs; the workspace then
 * needs no room for codes. */
size_t smx_fused_workspace_bytes(int model, size_t n_pairs, size_t dim);
int smx_score_backward_fused(int model, void* stream, const smx_plan_view* plan, float* table,
                             size_t n_rows, const int64_t* idx, const float* q1, const float* q2,
                             const float* score, const float* gscore, float* gq1, float* gq2,
                             size_t B, size_t K, size_t dim, const smx_score_params* params,
                             float* merged, float* m, float* v, const smx_opt_params* adam,
                             void* workspace, size_t workspace_bytes,
                             const void* fwd_codes, size_t fwd_codes_bytes);

/* Same pass for gradient rows that already exist in memory (what autograd hands
 * EmbedLookupFunc.backward): grad_rows [P, row_len] in pair order.  Replaces
 * merge_grad_list (embed_optimizer.py:45-48) and, when m, v, adam are given,
 * update_step (:208-252) on `table`. */
int smx_rows_backward(void* stream, const smx_plan_view* plan, const float* grad_rows,
                      size_t row_len, float* merged, float* table, float* m, float* v,
                      const smx_opt_params* adam, void* workspace, size_t workspace_bytes);

/* ---- negatives shared by the whole batch ------------------------------------------------------
 * Every training script of the reference runs with --share_negative: the sampler draws ONE list of K negative
 * ids per batch (smore/cpp_sampler/online_sampler.py:155-157), the model looks those K rows up once and scores
 * them against every query -- entity [1,K,row] against query [B,1,dim] (smore/models/kg_reasoning.py:349-355) --
 * and is_negative_mat masks the pairs that are true answers (smore/training/train_process.py:195-196; the mask
 * multiplies the logits, so it reaches the backward folded into gscore).  These entry points are the gather-fused
 * forms of that layout: ids [K] int64, score / gscore [B,K]; nothing of size B*K is built besides the logits.
 *   smx_score_forward_shared          score[b,k] = logit(table[ids[k]], q[b])       (as smx_score_forward)
 *   smx_score_backward_query_shared   gq1, gq2 [B,dim]                              (as smx_score_backward_query)
 *   smx_score_backward_entity_shared  the gradient of list position k is the sum over all B queries of
 *                                     d(gscore[b,k] * score[b,k]) / d row, summed in a fixed order (b ascending
 *                                     per wavefront, wavefronts in order), then
 *     plan == NULL: written to grad_rows[k,:] ([K, dim*mul]; the model's hook and the clamp mask of the entity
 *                   prologue applied -- what autograd hands EmbedLookupFunc.backward for the [1,K,row] lookup,
 *                   embed_optimizer.py:63-66).  The caller merges these rows with the step's other index streams:
 *                   grad_rows of smx_score_backward_entity_multi, or smx_rows_backward.
 *     plan != NULL: a plan built by smx_plan_build over exactly these K ids.  One result per DISTINCT id (a list
 *                   that holds an id twice sums both positions): merged[u,:] and / or the optimizer update of
 *                   table, m, v in place, as smx_score_backward_entity.
 * workspace of the three calls (may be NULL): smx_shared_workspace_bytes(model, B, K, dim)
 * bytes, 16-byte aligned.  Every model: room for the list's K rows side by side -- the query backward copies them
 * there first when the table spans 8 GiB or more (every query's workgroup reads all K rows; out of that much memory
 * each read is a page of its own), and always for the matrix products of COMPLEX and DISTMULT, whose entity side
 * also keeps its sums [K, n_q dim] there; COMPLEX with norm_on: the K rows scaled to unit-length halves as the
 * products' operand (without workspace the per-pair kernels run).
 * BETA_KL: given it (and rows of 16-byte aligned floats, dim a
 * multiple of 4), BetaE's entity-side terms -- three digammas and a log-beta per feature, dist_kernel.h:212-221 --
 * are evaluated once per shared row into the workspace instead of once per pair, and the pairs are a matrix product
 * on them (fp32 matrix instructions, fixed summation order); without it the per-pair kernels run (same results to
 * rounding: the product sums the divergence's four groups of terms separately); the entity side forms its sums
 * over the queries as a product too ([K,B] x [B,2 dim]) and finishes them row by row as before.  Each call fills the
 * workspace itself: nothing is carried from one call to the next.
 * Replaces dist_forward / dist_backward in the [1,K] x [B,1] layout (common_kernel.h:33-123) plus gather,
 * merge_grad_* and update_step as listed at smx_score_backward_entity. */
size_t smx_shared_workspace_bytes(int model, size_t B, size_t K, size_t dim);
int smx_score_forward_shared(int model, void* stream, const float* table, size_t n_rows, const int64_t* ids,
                             const float* q1, const float* q2, float* score, size_t B, size_t K, size_t dim,
                             const smx_score_params* params, int* err_flag, void* workspace,
                             size_t workspace_bytes);
int smx_score_backward_query_shared(int model, void* stream, const float* table, size_t n_rows, const int64_t* ids,
                                    const float* q1, const float* q2, const float* score, const float* gscore,
                                    float* gq1, float* gq2, size_t B, size_t K, size_t dim,
                                    const smx_score_params* params, void* workspace, size_t workspace_bytes);
int smx_score_backward_entity_shared(int model, void* stream, float* table, size_t n_rows, const int64_t* ids,
                                     const float* q1, const float* q2, const float* score, const float* gscore,
                                     size_t B, size_t K, size_t dim, const smx_score_params* params,
                                     const smx_plan_view* plan, float* grad_rows, float* merged, float* m, float* v,
                                     const smx_opt_params* adam, void* workspace, size_t workspace_bytes);

/* ---- sample loss ---------------------------------------------------------------------------
 * The loss between the scoring forward and its backward (smore/training/train_process.py:194-213)
 * and its gradient in one pass over the [B,K] negative logits:
 *   x = neg * mask (mask = is_negative_mat, may be NULL)
 *   s_b = sum_k softmax(x * temperature)_k logsigmoid(-x_k)   (temperature > 0; weights not differentiated, :197-199)
 *       | mean_k logsigmoid(-x_k)                             (temperature == 0, :200-201)
 *   pos_loss = -sum_b W_b logsigmoid(pos_b),  neg_loss = -sum_b W_b s_b,
 *   W_b = weight_b / sum(weight) (subsampling_weight, :203-207) or 1/B when weight is NULL (:208-211).
 * out_loss[2] (device) = {pos_loss, neg_loss}; gpos [B], gneg [B,K] = d((pos_loss + neg_loss) * scale) / d logit,
 * scale = 1/2/world_size (:213): gneg is the upstream gradient smx_score_backward_* consumes.
 * workspace: smx_sample_loss_workspace_bytes(B). */
size_t smx_sample_loss_workspace_bytes(size_t B);
int smx_sample_loss(void* stream, const float* pos, const float* neg, const float* mask,
                    const float* weight, size_t B, size_t K, double temperature, double scale,
                    float* out_loss, float* gpos, float* gneg, void* workspace, size_t workspace_bytes);

/* The same pass for callers that cannot allocate or pass a workspace: code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference.  The
 * 2 B + 1 floats of scratch live in a static device array of the library (one copy per device, 512 KiB,
 * held until the process ends); the call allocates nothing and gives the same bits as smx_sample_loss.
 * At most SMX_SAMPLE_LOSS_STATIC_MAX_QUERIES queries per call (more: SMX_ERR_SHAPE).  Every call on
 * a device shares that device's array: calls that overlap on one device (two streams, two threads)
 * race; calls on one stream are ordered.  The first call on a device asks the runtime for the array's
 * address (hipGetSymbolAddress), so make it before a stream capture begins. */
#define SMX_SAMPLE_LOSS_STATIC_MAX_QUERIES 65536
int smx_sample_loss_static(void* stream, const float* pos, const float* neg, const float* mask,
                           const float* weight, size_t B, size_t K, double temperature, double scale,
                           float* out_loss, float* gpos, float* gneg);

/* ---- evaluation against all entities --------------------------------------------------------
 * Filtered ranks of a query's answers among all n_rows entities (the test_all branch of
 * smore/training/train_process.py:112-160: logits of every entity, argsort, ranks of easy + hard
 * answers, minus the answers ranked before) without materialising or sorting the logit row: the
 * table is streamed once per one, two or four queries (as many as the row length allows) and every non-answer entity is counted against the answers
 * it ranks before.  Equal scores: the lower entity id ranks first.
 *   ans_id [B, A] int64, ans_count [B] int32: ans_count[b] <= A valid answers (easy and hard alike) per query.
 * smx_rank_answer_keys: ans_score [B, A] = the answers' logits, ans_key [B, A] = their order keys
 *   (larger key = ranked earlier; 0 in unused slots).
 * smx_rank_scan: ans_id / ans_key must be sorted by key, descending, within each query (unused slots
 *   last); filtered_rank [B, A] int64, 1-based, in that order (0 in unused slots).
 * workspace: smx_rank_workspace_bytes(B, A).  At most 2048 answers per query, n_rows <= 2^32. */
size_t smx_rank_workspace_bytes(size_t B, size_t A);
int smx_rank_answer_keys(int model, void* stream, const float* table, size_t n_rows, const float* q1,
                         const float* q2, size_t B, size_t dim, const smx_score_params* params,
                         const int64_t* ans_id, const int32_t* ans_count, size_t A, float* ans_score,
                         uint64_t* ans_key);
int smx_rank_scan(int model, void* stream, const float* table, size_t n_rows, const float* q1,
                  const float* q2, size_t B, size_t dim, const smx_score_params* params,
                  const int64_t* ans_id, const uint64_t* ans_key, const int32_t* ans_count, size_t A,
                  int64_t* filtered_rank, void* workspace, size_t workspace_bytes);

/* Evaluation against sampled candidates: the branch of test_step_mp taken when the evaluation set brings its own
 * negatives (smore/training/train_process.py:118-128, 141-147).  cand [B, C] int64: per query its candidates, the
 * first n_hard[b] of them its hard answers, -1 = padding.  As the reference does, a padding slot is scored as
 * entity 0 and -1e6 is added to its logit (:119-120, :123).
 *   logit [B, C]     (may be NULL) the biased logits, negative_logit of :123
 *   ranking [B, C]   position of candidate j in argsort(logit, descending) (:124-128); equal logits: the lower
 *                    candidate position first
 *   hard_rank [B, H] filtered rank, 1-based, of hard answer j < n_hard[b] in the order given: ranking[j] minus
 *                    the number of the query's hard answers ranked before it, plus 1 (:141-145); 0 in unused slots
 * One workgroup per query: scores, ranks by counting, no sort.  At most 4096 candidates per query, H <= C.
 * A candidate id other than -1 outside [0, n_rows) sets *err_flag (may be NULL) and is scored as entity 0. */
int smx_rank_candidates(int model, void* stream, const float* table, size_t n_rows, const float* q1,
                        const float* q2, size_t B, size_t dim, const smx_score_params* params,
                        const int64_t* cand, size_t C, const int32_t* n_hard, size_t H, float* logit,
                        int64_t* ranking, int64_t* hard_rank, int* err_flag);

/* The three evaluation calls for union queries: q1, q2 are [B, U, dim] (the U branch rows of a query adjacent, as
 * for smx_score_forward_union), and an entity's logit is the maximum over the branches -- the last line of every
 * custom_cal_logit (smore/models/box.py:163, vec.py:89, rotate.py:141, beta.py:307), which the evaluation loop
 * reaches through the same model call as training (train_process.py:112-123).  Everything else as above; the
 * ranks are those of the maximum logits, not the best of the branches' ranks.  U <= 4 (the scan keeps a query's
 * branch rows in registers: rows of more than 512 floats -- 256 for the two-halves models -- allow U <= 2).
 * U == 1 is the plain call. */
int smx_rank_answer_keys_union(int model, void* stream, const float* table, size_t n_rows, const float* q1,
                               const float* q2, size_t B, size_t U, size_t dim, const smx_score_params* params,
                               const int64_t* ans_id, const int32_t* ans_count, size_t A, float* ans_score,
                               uint64_t* ans_key);
int smx_rank_scan_union(int model, void* stream, const float* table, size_t n_rows, const float* q1,
                        const float* q2, size_t B, size_t U, size_t dim, const smx_score_params* params,
                        const int64_t* ans_id, const uint64_t* ans_key, const int32_t* ans_count, size_t A,
                        int64_t* filtered_rank, void* workspace, size_t workspace_bytes);
int smx_rank_candidates_union(int model, void* stream, const float* table, size_t n_rows, const float* q1,
                              const float* q2, size_t B, size_t U, size_t dim, const smx_score_params* params,
                              const int64_t* cand, size_t C, const int32_t* n_hard, size_t H, float* logit,
                              int64_t* ranking, int64_t* hard_rank, int* err_flag);

/* Plain row lookup out[k,:] = table[idx[k],:] (smore/common/embedding/embed_rw.py:74-75, the GPU
 * branch of EmbeddingReadOnly.read) for callers that need the rows themselves. */
int smx_gather_rows(void* stream, const float* table, size_t n_rows, size_t row_len,
                    const int64_t* idx, size_t n, float* out, int* err_flag);

#ifdef __cplusplus
}
#endif
#endif /* SMORE_AMD_H */
