// BetaE with negatives shared by the batch: the entity side of the KL divergence once per row.
//
// KL(Beta(e) || Beta(q)) per feature (smore/common/torchext/dist_kernel.h:207-266) is
//   [lgG(qa)+lgG(qb)-lgG(sq)] + [lgG(se)-lgG(ea)-lgG(eb)] + (ea-qa) psi(ea) + (eb-qb) psi(eb) + (sq-se) psi(se):
// three digammas and a log-beta of the ENTITY per (pair, feature), which is what makes the per-query kernels
// instruction-bound (smore/models/beta.py:303-308 through beta_dist.py).  With --share_negative
// (smore/cpp_sampler/online_sampler.py:155-157) the same K rows meet all B queries, so those entity terms are
// evaluated once per row into a side table -- K x dim evaluations instead of B x K x dim -- and a pair costs a
// handful of multiply-adds per feature on them.  The side table is several times the size of the rows, so it
// is reused from LDS: a workgroup stages a few rows' terms, and each of its wavefronts, holding one query in
// registers, scores that query against all of them.
//   forward:         score[b,k] = gamma - sum_d KL         (same per-feature expression and summation order
//                                                           as the per-query kernel: ModelOps<mBetaKL>::fwd)
//   query backward:  gqa[b,d] = sum_k c[b,k] ((psi(qa)-psi(sq)) - psi(ea_k) + psi(se_k)), same with b
//                                                          (ModelOps<mBetaKL>::bwd_q), rows in ascending order
// The entity side of the backward needs no special functions per pair at all (sums of c (e - q), one trigamma
// hook per finished row): it is shared_entity_kernel of smx_shared_impl.h as it stands.
#include "smx_common.h"
#include "smx_models.h"
#include "smx_wave.h"

namespace smx {

constexpr int kBsFwdWaves = 8;    // queries per workgroup of the forward (one per wavefront)
constexpr int kBsBwdWaves = 4;    // queries per workgroup of the query backward
constexpr int kBsFwdTile = 4;     // rows whose six term vectors are staged in LDS per turn (forward)
constexpr int kBsBwdTile = 8;     // rows whose three digamma vectors are staged per turn (query backward)
constexpr int kBsFwdChunk = 64;   // rows per workgroup of the forward
constexpr int kBsMaxDim = 512;    // two float4 columns per lane at most

typedef float bvec4 __attribute__((ext_vector_type(4)));

// terms of row ids[k]: forward {ea, eb, lgB(e), psi(ea), psi(eb), psi(se)} x dim, backward {psi(ea), psi(eb), psi(se)} x dim
// (ea, eb after the entity prologue clamp(x + add, lo, hi) when it is on); one wavefront per row.
template <bool FWD>
__global__ __launch_bounds__(256) void beta_row_terms_kernel(const float* __restrict__ table,
                                                             const long long* __restrict__ ids, int K, int dim,
                                                             unsigned long long n_rows, ScoreParams p,
                                                             float* __restrict__ terms, int* err) {
  const int lane = threadIdx.x & 63;
  const int k = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (k >= K) return;
  long long row = ids[k];
  if ((unsigned long long)row >= n_rows) {  // remember it, read row 0 instead (as every scorer of the library does)
    if (err && lane == 0) *err = 1;
    row = 0;
  }
  const float* e = table + (size_t)row * 2 * dim;
  constexpr int NV = FWD ? 6 : 3;
  float* out = terms + (size_t)k * NV * dim;
  for (int d = lane; d < dim; d += 64) {
    const float ea = reg_apply(e[d], p), eb = reg_apply(e[dim + d], p);
    float lb, pa, pb, ps;
    if constexpr (FWD) {
      beta_terms(ea, eb, lb, pa, pb, ps);
      out[d] = ea;
      out[dim + d] = eb;
      out[2 * dim + d] = lb;
      out[3 * dim + d] = pa;
      out[4 * dim + d] = pb;
      out[5 * dim + d] = ps;
    } else {
      digamma3(ea, eb, pa, pb, ps);
      out[d] = pa;
      out[dim + d] = pb;
      out[2 * dim + d] = ps;
    }
  }
}

template <int NIT, bool FWD>
__device__ __forceinline__ void load_beta_query(const float* __restrict__ q1, const float* __restrict__ q2, int b, int dim,
                                                int ncol, int lane, QBeta (&q)[NIT][4]) {
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    const int c = min(lane + 64 * it, ncol - 1);
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const float a = q1[(size_t)b * dim + c * 4 + v], bb = q2[(size_t)b * dim + c * 4 + v];
      q[it][v] = FWD ? ModelOps<mBetaKL>::prep_fwd(a, bb) : ModelOps<mBetaKL>::prep_bwd_q(a, bb);
    }
  }
}

// grid (ceil(B / 8), ceil(K / 64)); LDS: kBsFwdTile rows x 6 x dim floats
template <int NIT>
__global__ __launch_bounds__(kBsFwdWaves * 64) void beta_shared_forward_kernel(const float* __restrict__ terms,
                                                                               const float* __restrict__ q1,
                                                                               const float* __restrict__ q2,
                                                                               float* __restrict__ score, int B, int K,
                                                                               int dim, ScoreParams p) {
  extern __shared__ __align__(16) float tile[];
  const int lane = threadIdx.x & 63;
  const int wave = uniform(threadIdx.x >> 6);
  const int ncol = dim / 4;
  const int b_raw = blockIdx.x * kBsFwdWaves + wave;
  const int b = min(b_raw, B - 1);  // a wavefront past the last query computes along (it takes part in the barriers)
  const int k0 = blockIdx.y * kBsFwdChunk, k1 = min(K, k0 + kBsFwdChunk);
  QBeta q[NIT][4];
  load_beta_query<NIT, true>(q1, q2, b, dim, ncol, lane, q);
  // a thread's share of a tile travels through registers: the next tile is requested before this one is used
  constexpr int kPer = (kBsFwdTile * 6 * (kBsMaxDim / 4) + kBsFwdWaves * 64 - 1) / (kBsFwdWaves * 64);
  bvec4 next[kPer];
  auto request = [&](int kt) {
    const int n4 = min(kBsFwdTile, k1 - kt) * 6 * ncol;
    const bvec4* src = reinterpret_cast<const bvec4*>(terms + (size_t)kt * 6 * dim);
#pragma unroll
    for (int u = 0; u < kPer; ++u) {
      const int i = threadIdx.x + u * kBsFwdWaves * 64;
      if (i < n4) next[u] = src[i];
    }
  };
  request(k0);
  for (int kt = k0; kt < k1; kt += kBsFwdTile) {
    const int rows_here = min(kBsFwdTile, k1 - kt);
    __syncthreads();  // the previous rows have been used by every wavefront
#pragma unroll
    for (int u = 0; u < kPer; ++u) {
      const int i = threadIdx.x + u * kBsFwdWaves * 64;
      if (i < rows_here * 6 * ncol) reinterpret_cast<bvec4*>(tile)[i] = next[u];
    }
    __syncthreads();
    if (kt + kBsFwdTile < k1) request(kt + kBsFwdTile);
    for (int r = 0; r < rows_here; ++r) {
      const bvec4* t = reinterpret_cast<const bvec4*>(tile + (size_t)r * 6 * dim);
      float mine = 0.f;
#pragma unroll
      for (int it = 0; it < NIT; ++it) {
        const int c = min(lane + 64 * it, ncol - 1);
        const bvec4 ea = t[c], eb = t[ncol + c], lb = t[2 * ncol + c], pa = t[3 * ncol + c], pb = t[4 * ncol + c],
                    ps = t[5 * ncol + c];
        float a0 = 0.f;
#pragma unroll
        for (int v = 0; v < 4; ++v)
          a0 += (q[it][v].k + lb[v]) + (ea[v] - q[it][v].a) * pa[v] + (eb[v] - q[it][v].b) * pb[v] +
                ((q[it][v].a + q[it][v].b) - (ea[v] + eb[v])) * ps[v];
        mine += lane + 64 * it < ncol ? a0 : 0.f;
      }
      const float folded = wave_sum_last_f32(mine);
      if (lane == 63 && b_raw < B) score[(size_t)b * K + kt + r] = p.gamma - folded;
    }
  }
}

// Every workgroup walks all K rows (a query's gradient is one sum over them, rows ascending) for 4 / NIT queries: a
// query's columns are independent sums, so with two column groups two wavefronts share a query, one group each,
// and the grid is twice as long.  grid ceil(B * NIT / 4).  LDS: kBsBwdTile rows x 3 x dim floats
template <int NIT>
__global__ __launch_bounds__(kBsBwdWaves * 64) void beta_shared_backward_query_kernel(
    const float* __restrict__ terms, const float* __restrict__ q1, const float* __restrict__ q2,
    const float* __restrict__ gscore, float* __restrict__ gq1, float* __restrict__ gq2, int B, int K, int dim) {
  extern __shared__ __align__(16) float tile[];
  constexpr int kQueries = kBsBwdWaves / NIT;
  const int lane = threadIdx.x & 63;
  const int wave = uniform(threadIdx.x >> 6);
  const int ncol = dim / 4;
  const int b_raw = blockIdx.x * kQueries + wave / NIT;
  const int b = min(b_raw, B - 1);  // a wavefront past the last query computes along (it takes part in the barriers)
  const int my_col = lane + 64 * (wave % NIT);
  const int c = min(my_col, ncol - 1);
  QBeta q[4];
  float g1[4], g2[4];
#pragma unroll
  for (int v = 0; v < 4; ++v) {
    q[v] = ModelOps<mBetaKL>::prep_bwd_q(q1[(size_t)b * dim + c * 4 + v], q2[(size_t)b * dim + c * 4 + v]);
    g1[v] = g2[v] = 0.f;
  }
  // a thread's share of a tile travels through registers: the next tile is requested before this one is used
  // (64 is a multiple of the tile, so tiles never straddle a batch of upstream gradients)
  static_assert(64 % kBsBwdTile == 0, "tiles must not straddle a batch of 64 rows");
  constexpr int kPer = (kBsBwdTile * 3 * (kBsMaxDim / 4) + kBsBwdWaves * 64 - 1) / (kBsBwdWaves * 64);
  bvec4 next[kPer];
  auto request = [&](int kt) {
    const int n4 = min(kBsBwdTile, K - kt) * 3 * ncol;
    const bvec4* src = reinterpret_cast<const bvec4*>(terms + (size_t)kt * 3 * dim);
#pragma unroll
    for (int u = 0; u < kPer; ++u) {
      const int i = threadIdx.x + u * kBsBwdWaves * 64;
      if (i < n4) next[u] = src[i];
    }
  };
  request(0);
  for (int k64 = 0; k64 < K; k64 += 64) {
    const int n64 = min(64, K - k64);
    const float my_c0 = -gscore[(size_t)b * K + k64 + min(lane, n64 - 1)];  // d(gamma - KL) / d KL times the upstream gradient
    for (int kt = 0; kt < n64; kt += kBsBwdTile) {
      const int rows_here = min(kBsBwdTile, n64 - kt);
      __syncthreads();
#pragma unroll
      for (int u = 0; u < kPer; ++u) {
        const int i = threadIdx.x + u * kBsBwdWaves * 64;
        if (i < rows_here * 3 * ncol) reinterpret_cast<bvec4*>(tile)[i] = next[u];
      }
      __syncthreads();
      if (k64 + kt + kBsBwdTile < K) request(k64 + kt + kBsBwdTile);
      for (int r = 0; r < rows_here; ++r) {
        const float c0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(my_c0), kt + r));
        const bvec4* t = reinterpret_cast<const bvec4*>(tile + (size_t)r * 3 * dim);
        const bvec4 pa = t[c], pb = t[ncol + c], ps = t[2 * ncol + c];
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          g1[v] += c0 * (q[v].k - pa[v] + ps[v]);
          g2[v] += c0 * (q[v].l - pb[v] + ps[v]);
        }
      }
    }
  }
  if (b_raw >= B || my_col >= ncol) return;
  reinterpret_cast<bvec4*>(gq1 + (size_t)b * dim)[c] = bvec4{g1[0], g1[1], g1[2], g1[3]};
  reinterpret_cast<bvec4*>(gq2 + (size_t)b * dim)[c] = bvec4{g2[0], g2[1], g2[2], g2[3]};
}

// Whether the call can take these kernels: float4 columns, two per lane at most, aligned operands, room for the terms.
bool beta_shared_fits(size_t dim, const void* table, const void* q1, const void* q2, const void* workspace,
                      size_t workspace_bytes, size_t K, bool forward) {
  if (dim % 4 != 0 || dim > (size_t)kBsMaxDim || !workspace) return false;
  if (!aligned16(table) || !aligned16(q1) || !aligned16(q2) || !aligned16(workspace)) return false;
  return workspace_bytes >= K * (forward ? 6 : 3) * dim * sizeof(float);
}

int beta_shared_forward(hipStream_t st, const float* table, size_t n_rows, const long long* ids, const float* q1,
                        const float* q2, float* score, size_t B, size_t K, size_t dim, const ScoreParams& p, int* err,
                        float* terms) {
  hipLaunchKernelGGL(beta_row_terms_kernel<true>, dim3((unsigned)((K + 3) / 4)), dim3(256), 0, st, table, ids, (int)K,
                     (int)dim, (unsigned long long)n_rows, p, terms, err);
  const dim3 grid((unsigned)((B + kBsFwdWaves - 1) / kBsFwdWaves), (unsigned)((K + kBsFwdChunk - 1) / kBsFwdChunk));
  const size_t lds = (size_t)kBsFwdTile * 6 * dim * sizeof(float);
  if (dim <= 256)
    hipLaunchKernelGGL(beta_shared_forward_kernel<1>, grid, dim3(kBsFwdWaves * 64), lds, st, terms, q1, q2, score, (int)B,
                       (int)K, (int)dim, p);
  else
    hipLaunchKernelGGL(beta_shared_forward_kernel<2>, grid, dim3(kBsFwdWaves * 64), lds, st, terms, q1, q2, score, (int)B,
                       (int)K, (int)dim, p);
  return check_launch("score forward (shared negatives, beta_kl)");
}

int beta_shared_backward_query(hipStream_t st, const float* table, size_t n_rows, const long long* ids, const float* q1,
                               const float* q2, const float* gscore, float* gq1, float* gq2, size_t B, size_t K,
                               size_t dim, const ScoreParams& p, float* terms) {
  hipLaunchKernelGGL(beta_row_terms_kernel<false>, dim3((unsigned)((K + 3) / 4)), dim3(256), 0, st, table, ids, (int)K,
                     (int)dim, (unsigned long long)n_rows, p, terms, nullptr);
  const size_t lds = (size_t)kBsBwdTile * 3 * dim * sizeof(float);
  if (dim <= 256)
    hipLaunchKernelGGL(beta_shared_backward_query_kernel<1>, dim3((unsigned)((B + kBsBwdWaves - 1) / kBsBwdWaves)),
                       dim3(kBsBwdWaves * 64), lds, st, terms, q1, q2, gscore, gq1, gq2, (int)B, (int)K, (int)dim);
  else
    hipLaunchKernelGGL(beta_shared_backward_query_kernel<2>, dim3((unsigned)((2 * B + kBsBwdWaves - 1) / kBsBwdWaves)),
                       dim3(kBsBwdWaves * 64), lds, st, terms, q1, q2, gscore, gq1, gq2, (int)B, (int)K, (int)dim);
  return check_launch("score backward (query, shared negatives, beta_kl)");
}

}  // namespace smx
