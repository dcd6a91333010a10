/*
 * TEST INFRASTRUCTURE ONLY.
 *
 * CPU restatement (plain C) of the SMORE negative-sample scoring path:
 * gather -> distance forward/backward -> unique-merge of entity ids ->
 * segment sum -> lazy Adam.  It exists to check the HIP kernels and to be
 * timed as the host-core baseline; the shipped library never links it.
 *
 * Built by oracle/Makefile into oracle/liboracle.so.  Floating-point
 * functions exist in two precisions: *_f64 (the checker) and *_f32 (the
 * baseline that is timed), both generated from oracle_body.inc.
 *
 * Pinning status of each function (which independent check covers it) is
 * listed in oracle/oracle.py's module docstring.
 */
#define _DEFAULT_SOURCE
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

enum {
  ORC_L1 = 0,
  ORC_L2 = 1,
  ORC_BOX_OUT = 2,
  ORC_BOX_IN = 3,
  ORC_ROTATE = 4,
  ORC_BETA_KL = 5,
  ORC_COMPLEX = 6,
  ORC_DISTMULT = 7,
  ORC_BETA_L2 = 8,
  ORC_BETA_FISHER = 9,
  ORC_NUM_KINDS = 10
};

#define CAT_(a, b) a##b
#define CAT(a, b) CAT_(a, b)

#define REAL double
#define FN(name) CAT(name, _f64)
#define LOGF log
#define SINF sin
#define SQRTF sqrt
#define LGAMMAF lgamma_r
#include "oracle_body.inc"
#undef REAL
#undef FN
#undef LOGF
#undef SINF
#undef SQRTF
#undef LGAMMAF

#define REAL float
#define FN(name) CAT(name, _f32)
#define LOGF logf
#define SINF sinf
#define SQRTF sqrtf
#define LGAMMAF lgammaf_r
#include "oracle_body.inc"
#undef REAL
#undef FN
#undef LOGF
#undef SINF
#undef SQRTF
#undef LGAMMAF

/* ---- id merge: embedding/embed_optimizer.py:39-42 --------------------------
 * torch.unique(idx, return_inverse=True): uniq is sorted ascending and
 * strictly increasing, inverse[k] is the position of idx[k] in uniq.
 * Also returns, for the segment contract, the stable order of pairs grouped
 * by id (order[.]) and the first position of each segment (seg_start[0..U]).
 * Returns U. */
typedef struct {
  int64_t key;
  int64_t pos;
} orc_kp;

static int orc_kp_cmp(const void* a, const void* b) {
  const orc_kp* x = (const orc_kp*)a;
  const orc_kp* y = (const orc_kp*)b;
  if (x->key != y->key) return x->key < y->key ? -1 : 1;
  return x->pos < y->pos ? -1 : (x->pos > y->pos ? 1 : 0);
}

int64_t orc_merge_indices(const int64_t* idx, size_t p, int64_t* uniq, int64_t* inverse,
                          int64_t* order, int64_t* seg_start) {
  if (p == 0) {
    if (seg_start) seg_start[0] = 0;
    return 0;
  }
  orc_kp* kp = (orc_kp*)malloc(p * sizeof(orc_kp));
  for (size_t k = 0; k < p; ++k) {
    kp[k].key = idx[k];
    kp[k].pos = (int64_t)k;
  }
  qsort(kp, p, sizeof(orc_kp), orc_kp_cmp);
  int64_t u = -1;
  for (size_t k = 0; k < p; ++k) {
    if (k == 0 || kp[k].key != kp[k - 1].key) {
      ++u;
      uniq[u] = kp[k].key;
      if (seg_start) seg_start[u] = (int64_t)k;
    }
    inverse[kp[k].pos] = u;
    if (order) order[k] = kp[k].pos;
  }
  ++u;
  if (seg_start) seg_start[u] = (int64_t)p;
  free(kp);
  return u;
}
