// Negatives shared by the batch as matrix products: BetaE, ComplEx and DistMult.
//
// With --share_negative (smore/cpp_sampler/online_sampler.py:155-157) the same K rows meet all B queries.  For the
// models whose pair score is, or can be regrouped into, an inner product of something per row with something per
// query, the B x K pairs are then a matrix product with an operand shared along each axis -- the one shape on this
// path that the matrix cores fit (v_mfma_f32_32x32x2_f32: fp32 operands, fp32 accumulation in a fixed order).
//
// ComplEx, DistMult (smore/common/torchext/dist_kernel.h:187-204, 324-349): score = gamma + sum_j e[k,j] q[b,j], j over the
// row ([re | im] against [q1 | q2], or the D features of DistMult):
//   forward         [B, J] x [J, K]      (rows of the table gathered by the list's ids as the second operand)
//   query backward  gq = g [B, K] x E [K, J]
//   entity side     R = g^T [K, B] x [q1 | q2] [B, J]: the gradient row of list position k, finished (plan, optimizer)
//                   by shared_entity_kernel of smx_shared_impl.h
//
// BetaE: KL(Beta(e) || Beta(q)) per feature (dist_kernel.h:207-266) is
//   [lgG(qa)+lgG(qb)-lgG(sq)] + [lgG(se)-lgG(ea)-lgG(eb)] + (ea-qa) psi(ea) + (eb-qb) psi(eb) + (sq-se) psi(se):
// three digammas and a log-beta of the ENTITY per (pair, feature), which is what makes the per-query kernels
// instruction-bound (smore/models/beta.py:303-308 through beta_dist.py).  Regrouped by what each term depends on,
//   KL[b,k] = Qk[b] + Ek[k] + sum_d qa[b,d] T[k,d] + sum_d qb[b,d] T[k,D+d]
//     T[k,d] = psi(se)-psi(ea),  T[k,D+d] = psi(se)-psi(eb)                       (one row of 2D floats per shared row)
//     Ek[k]  = sum_d [lgG(se)-lgG(ea)-lgG(eb)] + ea psi(ea) + eb psi(eb) - se psi(se)
//     Qk[b]  = sum_d lgG(qa)+lgG(qb)-lgG(sq)
// the special functions are evaluated K x D + B x D times instead of B x K x D, and what is left per pair is the
// product [B, 2D] x [2D, K] with T in the place of the rows.  The query backward is the other product with T,
//   gqa[b,d] = (psi(qa)-psi(sq)) sum_k c[b,k] + sum_k c[b,k] T[k,d]            (c = -upstream gradient; same with b),
// and the entity side (ModelOps<mBetaKL>::bwd_e sums c (ea - qa) and c (eb - qb) over the queries) is
//   S1[k,d] = ea[k,d] C[k] - R[k,d],  S2[k,d] = eb[k,d] C[k] - R[k,D+d],  C[k] = sum_b c[b,k],  R = c^T x [q1 | q2],
// turned into the gradient row (trigamma hook, clamp mask, optimizer) by shared_entity_kernel.  The sums are those of
// ModelOps<mBetaKL>::fwd / bwd_q / bwd_e taken in another order: the groups of terms are summed separately, which
// costs some of the tolerance's headroom (measured in the tests), not the bar.
#include "smx_common.h"
#include "smx_models.h"
#include "smx_wave.h"

namespace smx {

typedef float facc16 __attribute__((ext_vector_type(16)));

// ---- the terms of the shared rows: T [K][2D], then (forward) Ek [K]; one wavefront per row ------------------
template <bool FWD>
__global__ __launch_bounds__(256) void beta_row_terms_kernel(const float* __restrict__ table,
                                                             const long long* __restrict__ ids, int K, int dim,
                                                             unsigned long long n_rows, ScoreParams p,
                                                             float* __restrict__ T, float* __restrict__ Ek, int* err) {
  const int lane = threadIdx.x & 63;
  const int k = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (k >= K) return;
  long long row = ids[k];
  if ((unsigned long long)row >= n_rows) {  // remember it, read row 0 instead (as every scorer of the library does)
    if (err && lane == 0) *err = 1;
    row = 0;
  }
  const float* e = table + (size_t)row * 2 * dim;
  float* out = T + (size_t)k * 2 * dim;
  float mine = 0.f;
  for (int d = lane; d < dim; d += 64) {
    const float ea = reg_apply(e[d], p), eb = reg_apply(e[dim + d], p);
    float lb, pa, pb, ps;
    if constexpr (FWD) {
      beta_terms(ea, eb, lb, pa, pb, ps);
      mine += (lb + ea * pa) + (eb * pb - (ea + eb) * ps);
    } else {
      digamma3(ea, eb, pa, pb, ps);
    }
    out[d] = ps - pa;
    out[dim + d] = ps - pb;
  }
  if constexpr (FWD) {
    const float total = wave_sum_last_f32(mine);
    if (lane == 63) Ek[k] = total;
  }
}

// Qk [B]: one wavefront per query
__global__ __launch_bounds__(256) void beta_query_terms_kernel(const float* __restrict__ q1, const float* __restrict__ q2,
                                                               int B, int dim, float* __restrict__ Qk) {
  const int lane = threadIdx.x & 63;
  const int b = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (b >= B) return;
  float mine = 0.f;
  for (int d = lane; d < dim; d += 64) mine += ModelOps<mBetaKL>::prep_fwd(q1[(size_t)b * dim + d], q2[(size_t)b * dim + d]).k;
  const float total = wave_sum_last_f32(mine);
  if (lane == 63) Qk[b] = total;
}

// ---- the matrix products ------------------------------------------------------------------------------------
// A 32 x 32 tile of the result is formed by walking the inner dimension two at a time with
// v_mfma_f32_32x32x2_f32.  Operand layout of the instruction: lane l supplies A[l % 32][l / 32] and B[l / 32][l % 32];
// of the 16 accumulators of lane l, number r is the element (8 (r / 4) + 4 (l / 32) + r % 4, l % 32).
__device__ __forceinline__ int acc_row(int r, int lane) { return 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3); }

// The four wavefronts of a workgroup share one tile: each walks a quarter of the inner dimension, the partial tiles
// are added through LDS in wavefront order, the first wavefront finishes (a tile alone would leave a SIMD one
// wavefront whose loads nothing hides).
__device__ __forceinline__ void combine_tiles(facc16& acc, float* part, int wave, int lane) {
  if (wave > 0) {
#pragma unroll
    for (int r = 0; r < 16; ++r) part[((wave - 1) * 16 + r) * 64 + lane] = acc[r];
  }
  __syncthreads();
  if (wave == 0) {
#pragma unroll
    for (int w = 1; w < 4; ++w)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[r] += part[((w - 1) * 16 + r) * 64 + lane];
  }
}

// What the three products need to know about a call.  BETA: the second operand's rows are rows of T, else rows of
// the table found through the list's ids; nq = query tensors (the inner dimension is nq * dim features).
struct GemmArgs {
  const float* rows;       // T [K][2 dim] (BETA) or the table
  const long long* ids;    // [K] (not BETA); null: `rows` holds the K rows themselves, in list order
  unsigned long long n_rows;
  const float* q1;
  const float* q2;
  const float* gscore;     // [B, K]
  const float* Ek;         // BETA forward
  const float* Qk;
  float* out1;             // score; gq1; R
  float* out2;             // gq2; C
  int B, K, dim, nq;
  float gamma;
  int* err;
};

template <bool BETA>
__device__ __forceinline__ const float* shared_row(const GemmArgs& A, int k, int& bad) {
  if constexpr (BETA) {
    return A.rows + (size_t)k * 2 * A.dim;
  } else {
    if (!A.ids) return A.rows + (size_t)k * A.nq * A.dim;  // uniform
    long long row = A.ids[k];
    if ((unsigned long long)row >= A.n_rows) {  // remember it, read row 0 instead (as every scorer of the library does)
      bad = 1;
      row = 0;
    }
    return A.rows + (size_t)row * A.nq * A.dim;
  }
}

// score[b,k] = gamma -/+ (... + sum_j q[b,j] row_k[j]), j over the nq * dim features ([q1 | q2] against a row).
// Both operands have the inner dimension contiguous, so a lane's operand values lie along its own row: it reads
// four neighbouring features per 16-byte load and feeds them to four instructions (8-byte loads for two
// instructions took 26 us where this takes 21, ComplEx at B = 512, K = 1024, D = 400: the loads of a wavefront touch
// 64 different lines either way).  The units of eight features are dealt out to the four wavefronts in contiguous
// quarters.
template <bool BETA>
__global__ __launch_bounds__(256) void shared_forward_gemm_kernel(GemmArgs A) {
  __shared__ float part[3 * 16 * 64];
  const int lane = threadIdx.x & 63;
  const int wave = uniform(threadIdx.x >> 6);
  const int B = A.B, K = A.K, dim = A.dim;
  const int tiles_k = (K + 31) / 32;
  const int tile = blockIdx.x;
  const int b0 = (tile / tiles_k) * 32, k0 = (tile % tiles_k) * 32;
  const int half = lane >> 5, col = lane & 31;
  const int my_b = min(b0 + col, B - 1), my_k = min(k0 + col, K - 1);  // rows past the end repeat the last one; never stored
  int bad = 0;
  // a unit of eight features: lanes 0-31 supply features 8 u .. 8 u + 3 of their row, lanes 32-63 features
  // 8 u + 4 .. 8 u + 7, one 16-byte load each; instruction s of the unit's four takes element s of both
  const float* t_row = shared_row<BETA>(A, my_k, bad);
  const float* a1_row = A.q1 + (size_t)my_b * dim;
  const float* a2_row = A.nq == 2 ? A.q2 + (size_t)my_b * dim : a1_row;
  if (bad && A.err) *A.err = 1;
  const int J = A.nq * dim;            // the inner dimension, a multiple of four
  const int UT = (J + 7) / 8;          // units
  const int per = (UT + 3) / 4;
  const int u_lo = wave * per, u_hi = min(UT, u_lo + per);
  typedef float f4 __attribute__((ext_vector_type(4)));
  const f4 zero4 = {0.f, 0.f, 0.f, 0.f};
  auto ld_a = [&](int ui) -> f4 {
    const int f = 8 * min(ui, UT - 1) + 4 * half;
    if (f >= J) return zero4;  // the second half of a last unit of four features
    return *reinterpret_cast<const f4*>(f < dim ? a1_row + f : a2_row + (f - dim));
  };
  auto ld_t = [&](int ui) -> f4 {
    const int f = 8 * min(ui, UT - 1) + 4 * half;
    return f >= J ? zero4 : *reinterpret_cast<const f4*>(t_row + f);
  };
  facc16 acc = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  // four units at a time, the next four requested before these are used (requests past the end repeat the last unit)
  f4 av[4], tv[4], an[4], tn[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    av[u] = ld_a(u_lo + u);
    tv[u] = ld_t(u_lo + u);
  }
  for (int g = u_lo; g < u_hi; g += 4) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      an[u] = ld_a(g + 4 + u);
      tn[u] = ld_t(g + 4 + u);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (g + u < u_hi) {  // uniform
#pragma unroll
        for (int e = 0; e < 4; ++e) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av[u][e], tv[u][e], acc, 0, 0, 0);
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      av[u] = an[u];
      tv[u] = tn[u];
    }
  }
  combine_tiles(acc, part, wave, lane);
  const int k = k0 + col;
  if (wave != 0 || k >= K) return;
  const float ek = BETA ? A.Ek[k] : 0.f;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int b = b0 + acc_row(r, lane);
    if (b < B) A.out1[(size_t)b * K + k] = BETA ? A.gamma - ((A.Qk[b] + ek) + acc[r]) : A.gamma + acc[r];
  }
}

// gq[b,n] = sum_k c[b,k] row_k[n] (+ kq[b,n] sum_k c[b,k] for BETA), n over the nq * dim features (n < dim: gq1, else
// gq2), c = -gscore (BETA) or gscore.  The lanes of a tile's A operand also add up what they load: the row sums of
// c come for free.  Each of the four wavefronts walks a quarter of the list, a multiple of eight rows: four
// instructions take eight rows, lanes 0-31 supplying rows kk .. kk+3 and lanes 32-63 rows kk+4 .. kk+7 (one 16-byte
// load of coefficients per lane when the rows of gscore are 16-byte aligned).
template <bool BETA>
__global__ __launch_bounds__(256) void shared_backward_query_gemm_kernel(GemmArgs A) {
  __shared__ float part[3 * 16 * 64];
  __shared__ float part_c[3 * 64];
  const int lane = threadIdx.x & 63;
  const int wave = uniform(threadIdx.x >> 6);
  const int B = A.B, K = A.K, dim = A.dim;
  const int width = A.nq * dim;
  const int tiles_n = (width + 31) / 32;
  const int tile = blockIdx.x;
  const int b0 = (tile / tiles_n) * 32, n0 = (tile % tiles_n) * 32;
  const int half = lane >> 5, col = lane & 31;
  const int my_b = min(b0 + col, B - 1);
  const int my_n = min(n0 + col, width - 1);
  const float* a = A.gscore + (size_t)my_b * K;
  constexpr float kSign = BETA ? -1.f : 1.f;
  facc16 acc = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  float c_sum = 0.f;
  const int per = ((K + 31) / 32) * 8;
  const int k_lo = wave * per, k_hi = min(K, k_lo + per);
  const bool wide = (K & 3) == 0 && (reinterpret_cast<unsigned long long>(A.gscore) & 15ull) == 0ull;
  // the next eight rows are requested before these are used; a request past the end of the stretch repeats the
  // list's last row with coefficient 0
  float cv[4], tv[4], cn[4], tn[4];
  int bad = 0;
  auto request = [&](float (&c)[4], float (&tt)[4], int kk0) {
    const int k4 = kk0 + 4 * half;
    if (wide && k4 + 3 < k_hi) {  // (k_hi is a multiple of 4 here: all four rows or none)
      const float4 g = *reinterpret_cast<const float4*>(a + k4);
      c[0] = kSign * g.x;
      c[1] = kSign * g.y;
      c[2] = kSign * g.z;
      c[3] = kSign * g.w;
    } else {
#pragma unroll
      for (int u = 0; u < 4; ++u) c[u] = k4 + u < k_hi ? kSign * a[min(k4 + u, K - 1)] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) tt[u] = shared_row<BETA>(A, min(k4 + u, K - 1), bad)[my_n];
  };
  request(cv, tv, k_lo);
  for (int kk = k_lo; kk < k_hi; kk += 8) {
    request(cn, tn, kk + 8);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (kk + u < k_hi) {  // uniform (rows kk+4+u past the end carry coefficient 0)
        c_sum += cv[u];
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(cv[u], tv[u], acc, 0, 0, 0);
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      cv[u] = cn[u];
      tv[u] = tn[u];
    }
  }
  c_sum += __shfl_xor(c_sum, 32);  // row my_b: both halves of every eight rows
  if (wave > 0) part_c[(wave - 1) * 64 + lane] = c_sum;
  combine_tiles(acc, part, wave, lane);
  if (wave != 0) return;
#pragma unroll
  for (int w = 1; w < 4; ++w) c_sum += part_c[(w - 1) * 64 + lane];
  const int n = n0 + col;
  const int d = n < dim ? n : n - dim;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int row = acc_row(r, lane);
    const float s = __shfl(c_sum, row);
    const int b = b0 + row;
    if (b < B && n < width) {
      float v = acc[r];
      if constexpr (BETA) {
        const QBeta q = ModelOps<mBetaKL>::prep_bwd_q(A.q1[(size_t)b * dim + d], A.q2[(size_t)b * dim + d]);
        v += (n < dim ? q.k : q.l) * s;
      }
      (n < dim ? A.out1 : A.out2)[(size_t)b * dim + d] = v;
    }
  }
}

// R[k,n] = sum_b c[b,k] q[b,n], n over the nq * dim features of [q1 | q2], and C[k] = sum_b c[b,k] (BETA), left in the
// workspace for shared_entity_kernel.  Both operands are read along their contiguous dimension (lane l:
// c[b + l / 32][k0 + l % 32] and q[b + l / 32][n0 + l % 32]); each of the four wavefronts walks a quarter of the queries.
template <bool BETA>
__global__ __launch_bounds__(256) void shared_entity_gemm_kernel(GemmArgs A) {
  __shared__ float part[3 * 16 * 64];
  __shared__ float part_c[3 * 64];
  const int lane = threadIdx.x & 63;
  const int wave = uniform(threadIdx.x >> 6);
  const int B = A.B, K = A.K, dim = A.dim;
  const int width = A.nq * dim;
  const int tiles_n = (width + 31) / 32;
  const int tile = blockIdx.x;
  const int k0 = (tile / tiles_n) * 32, n0 = (tile % tiles_n) * 32;
  const int half = lane >> 5, col = lane & 31;
  const int my_k = min(k0 + col, K - 1);
  const int my_n = min(n0 + col, width - 1);
  const float* a = A.gscore + my_k;
  const float* t = my_n < dim ? A.q1 + my_n : A.q2 + (my_n - dim);
  constexpr float kSign = BETA ? -1.f : 1.f;
  facc16 acc = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  float c_sum = 0.f;
  const int per = ((B + 31) / 32) * 8;  // a multiple of eight queries: four instructions
  const int b_lo = wave * per, b_hi = min(B, b_lo + per);
  float cv[4], tv[4], cn[4], tn[4];
  auto request = [&](float (&c)[4], float (&tt)[4], int bb0) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int b = bb0 + 2 * u + half;
      const int bc = min(b, B - 1);
      c[u] = b < b_hi ? kSign * a[(size_t)bc * K] : 0.f;
      tt[u] = t[(size_t)bc * dim];
    }
  };
  request(cv, tv, b_lo);
  for (int bb = b_lo; bb < b_hi; bb += 8) {
    request(cn, tn, bb + 8);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (bb + 2 * u < b_hi) {  // uniform (an odd query past the end carries coefficient 0)
        c_sum += cv[u];
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(cv[u], tv[u], acc, 0, 0, 0);
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      cv[u] = cn[u];
      tv[u] = tn[u];
    }
  }
  c_sum += __shfl_xor(c_sum, 32);  // list position my_k: even queries of the stretch + odd ones
  if (wave > 0) part_c[(wave - 1) * 64 + lane] = c_sum;
  combine_tiles(acc, part, wave, lane);
  if (wave != 0) return;
#pragma unroll
  for (int w = 1; w < 4; ++w) c_sum += part_c[(w - 1) * 64 + lane];
  if (BETA && n0 == 0 && half == 0 && k0 + col < K) A.out2[k0 + col] = c_sum;
  const int n = n0 + col;
  if (n >= width) return;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int k = k0 + acc_row(r, lane);
    if (k < K) A.out1[(size_t)k * width + n] = acc[r];
  }
}

// ---- the K rows of the list side by side, as the products' second operand -------------------------------------
// UNIT (ComplEx with unit-length halves, width = 2 dim): out [K][2 dim], row k = [re / max(|re|, eps) |
// im / max(|im|, eps)] of table row ids[k]; DistMult with unit-length rows, width = dim: e / max(|e|, eps).  One
// wavefront per row.
// Not UNIT: out [K][width], row k = table row ids[k] as it is.  The query backward reads 128-byte pieces of all K
// rows in each of its tiles.  Through the ids every such piece is a load that waits for another (the id, then the
// row), K of them in a row per wavefront; from the copy the addresses are arithmetic and the rows one stretch of
// memory (B = 512, K = 1024, D = 400: ComplEx 54 -> 4 + 24 us, DistMult 43 -> 4 + 18, whatever the table's size).
template <bool UNIT>
__global__ __launch_bounds__(256) void list_rows_kernel(const float* __restrict__ table, const long long* __restrict__ ids,
                                                        int K, int dim, int width, unsigned long long n_rows,
                                                        float* __restrict__ En, int* err) {
  const int lane = threadIdx.x & 63;
  const int k = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (k >= K) return;
  long long row = ids[k];
  if ((unsigned long long)row >= n_rows) {
    if (err && lane == 0) *err = 1;
    row = 0;
  }
  const float* e = table + (size_t)row * width;
  float* out = En + (size_t)k * width;
  if constexpr (!UNIT) {
    typedef float f4 __attribute__((ext_vector_type(4)));  // (width is a multiple of four, the rows 16-byte aligned)
    for (int c = lane; c < width / 4; c += 64) reinterpret_cast<f4*>(out)[c] = reinterpret_cast<const f4*>(e)[c];
    return;
  }
  const bool two = width == 2 * dim;  // ComplEx; DistMult: the row is its only half
  float s1 = 0.f, s2 = 0.f;
  for (int d = lane; d < dim; d += 64) {
    s1 = __builtin_fmaf(e[d], e[d], s1);
    if (two) s2 = __builtin_fmaf(e[dim + d], e[dim + d], s2);
  }
  const float i1 = inv_norm(wave_sum_f32(s1)), i2 = inv_norm(wave_sum_f32(s2));
  for (int d = lane; d < dim; d += 64) {
    out[d] = e[d] * i1;
    if (two) out[dim + d] = e[dim + d] * i2;
  }
}

// ---- host side ----------------------------------------------------------------------------------------------
// out [K][width] = table rows ids[k], width a multiple of four floats, everything 16-byte aligned
int shared_list_rows(hipStream_t st, const float* table, size_t n_rows, const long long* ids, size_t K, size_t width,
                     float* out) {
  hipLaunchKernelGGL(list_rows_kernel<false>, dim3((unsigned)((K + 3) / 4)), dim3(256), 0, st, table, ids, (int)K, 0,
                     (int)width, (unsigned long long)n_rows, out, nullptr);
  return check_launch("rows of the shared list, side by side");
}

static bool is_inner(int model) { return model == mComplex || model == mDistmult; }

// floats of workspace a call of the model needs: forward / query backward, and the entity side
// (norm: ComplEx with unit-length halves, whose scaled rows stand in the workspace for the first two)
size_t shared_gemm_workspace_floats(int model, size_t B, size_t K, size_t dim, bool entity, bool norm) {
  if (model == mBetaKL) return entity ? K * (2 * dim + 1) : K * (2 * dim + 1) + B;
  if (is_inner(model)) return entity || norm ? K * (size_t)model_nq(model) * dim : 0;
  return 0;
}

// Whether the call can take these kernels: a model with a product form, float4-aligned operands, room in the workspace.
bool shared_gemm_fits(int model, size_t dim, const void* table, const void* q1, const void* q2, const void* workspace,
                      size_t workspace_bytes, size_t B, size_t K, bool entity, bool norm) {
  if (model != mBetaKL && !is_inner(model)) return false;
  if (dim % 4 != 0 || !aligned16(table) || !aligned16(q1) || (model_nq(model) == 2 && !aligned16(q2))) return false;
  const size_t need = shared_gemm_workspace_floats(model, B, K, dim, entity, norm) * sizeof(float);
  if (need == 0) return true;
  return workspace && aligned16(workspace) && workspace_bytes >= need;
}

static GemmArgs gemm_args(int model, const float* table, size_t n_rows, const long long* ids, const float* q1,
                          const float* q2, const float* gscore, size_t B, size_t K, size_t dim, float gamma, int* err) {
  GemmArgs A{};
  A.rows = table;
  A.ids = ids;
  A.n_rows = n_rows;
  A.q1 = q1;
  A.q2 = q2;
  A.gscore = gscore;
  A.B = (int)B;
  A.K = (int)K;
  A.dim = (int)dim;
  A.nq = model_nq(model);
  A.gamma = gamma;
  A.err = err;
  return A;
}

int shared_gemm_forward(int model, hipStream_t st, const float* table, size_t n_rows, const long long* ids,
                        const float* q1, const float* q2, float* score, size_t B, size_t K, size_t dim,
                        const ScoreParams& p, int* err, float* workspace) {
  GemmArgs A = gemm_args(model, table, n_rows, ids, q1, q2, nullptr, B, K, dim, p.gamma, err);
  A.out1 = score;
  const unsigned tiles = (unsigned)(((B + 31) / 32) * ((K + 31) / 32));
  if (model == mBetaKL) {
    float* T = workspace;
    float* Ek = T + K * 2 * dim;
    float* Qk = Ek + K;
    hipLaunchKernelGGL(beta_row_terms_kernel<true>, dim3((unsigned)((K + 3) / 4)), dim3(256), 0, st, table, ids, (int)K,
                       (int)dim, (unsigned long long)n_rows, p, T, Ek, err);
    hipLaunchKernelGGL(beta_query_terms_kernel, dim3((unsigned)((B + 3) / 4)), dim3(256), 0, st, q1, q2, (int)B, (int)dim, Qk);
    A.rows = T;
    A.Ek = Ek;
    A.Qk = Qk;
    hipLaunchKernelGGL(shared_forward_gemm_kernel<true>, dim3(tiles), dim3(256), 0, st, A);
  } else {
    if (p.norm_on) {
      hipLaunchKernelGGL(list_rows_kernel<true>, dim3((unsigned)((K + 3) / 4)), dim3(256), 0, st, table, ids, (int)K,
                         (int)dim, model_nq(model) * (int)dim, (unsigned long long)n_rows, workspace, err);
      A.rows = workspace;
      A.ids = nullptr;
    }
    hipLaunchKernelGGL(shared_forward_gemm_kernel<false>, dim3(tiles), dim3(256), 0, st, A);
  }
  return check_launch("score forward (shared negatives, matrix product)");
}

int shared_gemm_backward_query(int model, hipStream_t st, const float* table, size_t n_rows, const long long* ids,
                               const float* q1, const float* q2, const float* gscore, float* gq1, float* gq2, size_t B,
                               size_t K, size_t dim, const ScoreParams& p, float* workspace, size_t workspace_bytes) {
  GemmArgs A = gemm_args(model, table, n_rows, ids, q1, q2, gscore, B, K, dim, p.gamma, nullptr);
  A.out1 = gq1;
  A.out2 = gq2;
  const unsigned tiles = (unsigned)(((B + 31) / 32) * ((model_nq(model) * dim + 31) / 32));
  if (model == mBetaKL) {
    float* T = workspace;
    hipLaunchKernelGGL(beta_row_terms_kernel<false>, dim3((unsigned)((K + 3) / 4)), dim3(256), 0, st, table, ids, (int)K,
                       (int)dim, (unsigned long long)n_rows, p, T, nullptr, nullptr);
    A.rows = T;
    hipLaunchKernelGGL(shared_backward_query_gemm_kernel<true>, dim3(tiles), dim3(256), 0, st, A);
  } else {
    const int width = model_nq(model) * (int)dim;
    const dim3 grid((unsigned)((K + 3) / 4));
    if (p.norm_on) {  // (scaled again rather than kept: the entity side of the previous step has used the workspace since)
      hipLaunchKernelGGL(list_rows_kernel<true>, grid, dim3(256), 0, st, table, ids, (int)K, (int)dim, width,
                         (unsigned long long)n_rows, workspace, nullptr);
      A.rows = workspace;
      A.ids = nullptr;
    } else if (workspace && aligned16(workspace) && workspace_bytes >= K * (size_t)width * sizeof(float) && K >= 64) {
      // the rows side by side first (see list_rows_kernel)
      hipLaunchKernelGGL(list_rows_kernel<false>, grid, dim3(256), 0, st, table, ids, (int)K, (int)dim, width,
                         (unsigned long long)n_rows, workspace, nullptr);
      A.rows = workspace;
      A.ids = nullptr;
    }
    hipLaunchKernelGGL(shared_backward_query_gemm_kernel<false>, dim3(tiles), dim3(256), 0, st, A);
  }
  return check_launch("score backward (query, shared negatives, matrix product)");
}

// R [K][nq dim] (and C [K] for beta_kl) for the entity side; workspace: shared_gemm_workspace_floats(.., true)
int shared_gemm_entity_sums(int model, hipStream_t st, const float* q1, const float* q2, const float* gscore, size_t B,
                            size_t K, size_t dim, float* workspace) {
  GemmArgs A = gemm_args(model, nullptr, 0, nullptr, q1, q2, gscore, B, K, dim, 0.f, nullptr);
  const size_t width = (size_t)model_nq(model) * dim;
  A.out1 = workspace;
  A.out2 = workspace + K * width;
  const unsigned tiles = (unsigned)(((K + 31) / 32) * ((width + 31) / 32));
  if (model == mBetaKL)
    hipLaunchKernelGGL(shared_entity_gemm_kernel<true>, dim3(tiles), dim3(256), 0, st, A);
  else
    hipLaunchKernelGGL(shared_entity_gemm_kernel<false>, dim3(tiles), dim3(256), 0, st, A);
  return check_launch("entity backward (shared negatives, sums as a matrix product)");
}

}  // namespace smx
