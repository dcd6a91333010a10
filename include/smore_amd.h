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

int smx_version(void);
const char* smx_last_error(void);

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

#ifdef __cplusplus
}
#endif
#endif /* SMORE_AMD_H */
