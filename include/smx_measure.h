/*
 * smx_measure -- entry points of libsmore_amd.so that exist for measurement only.  Not part of the drop-in C ABI
 * of smore_amd.h: no caller of the scoring path needs them, and what they leave behind is not a training step.
 */
#ifndef SMX_MEASURE_H
#define SMX_MEASURE_H

#include "smore_amd.h"

#ifdef __cplusplus
extern "C" {
#endif

/* No counterpart in the reference.  smx_score_backward_fused with only some of its kernels launched, so that a
 * harness can bracket one half of the call with events by itself:
 *   parts bit 0   the query-gradient kernel (with the rows of ids that occur once)
 *   parts bit 1   the entity pass (segment, tile and fix-up kernels)
 * parts = 3 is smx_score_backward_fused.  With 1 or 2 the step is INCOMPLETE: rows of the other half are not
 * updated and, with 2, the query gradients are not written.  The choice is an argument of the call: nothing is
 * remembered, no other call or caller is affected. */
int smx_measure_backward_fused(int parts, int model, void* stream, const smx_plan_view* plan, float* table,
                               size_t n_rows, const int64_t* idx, const float* q1, const float* q2,
                               const float* score, const float* gscore, float* gq1, float* gq2, size_t B, size_t K,
                               size_t dim, const smx_score_params* params, float* merged, float* m, float* v,
                               const smx_opt_params* adam, void* workspace, size_t workspace_bytes,
                               const void* fwd_codes, size_t fwd_codes_bytes);

/* No counterpart in the reference.  Two HIP events (hipEvent_t, created with timing) that the NEXT
 * smx_score_backward_fused / smx_measure_backward_fused call of this host thread records on the caller's stream
 * immediately before and after its query-gradient kernel, so that a harness can time that kernel in its place
 * inside the call (the entity pass still follows it) instead of bracketing a call that launches nothing else.
 * The events are used once; NULL, NULL clears a pair that was set and not used. */
int smx_measure_query_kernel_events(void* before, void* after);

/* No counterpart in the reference.  smx_plan_build with the two knobs a test needs to see a plan give up while
 * every kernel still ends normally:
 *   spin_limit    polls a workgroup of the sort makes before it stops waiting for another one (the library
 *                 uses 2^22); 0 makes a workgroup give up the first time it would have to wait
 *   force_abort   != 0: the build starts with its "a workgroup gave up" word already set, so every pass leaves
 *                 without writing (also for inputs small enough for the one-workgroup build)
 * A build that gave up leaves *err_flag = 2 and *n_uniq = -1; the kernels that read a plan look at n_uniq first
 * and do nothing for such a plan. */
int smx_measure_plan_build(void* stream, const int64_t* idx, size_t n_pairs, size_t n_rows, void* workspace,
                           size_t workspace_bytes, int32_t* order, int32_t* sorted_ids, int32_t* seg_of_pos,
                           int64_t* uniq, int32_t* seg_start, int64_t* inverse, int32_t* pair_seg, int32_t* n_uniq,
                           int* err_flag, unsigned spin_limit, int force_abort);

#ifdef __cplusplus
}
#endif
#endif /* SMX_MEASURE_H */
