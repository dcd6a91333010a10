// BetaE with negatives shared by the batch: the entity side of the KL divergence once per row, the pairs as a
// matrix product.
//
// KL(Beta(e) || Beta(q)) per feature (smore/common/torchext/dist_kernel.h:207-266) is
//   [lgG(qa)+lgG(qb)-lgG(sq)] + [lgG(se)-lgG(ea)-lgG(eb)] + (ea-qa) psi(ea) + (eb-qb) psi(eb) + (sq-se) psi(se):
// three digammas and a log-beta of the ENTITY per (pair, feature), which is what makes the per-query kernels
// instruction-bound (smore/models/beta.py:303-308 through beta_dist.py).  With --share_negative
// (smore/cpp_sampler/online_sampler.py:155-157) the same K rows meet all B queries.  Regrouped by what each
// term depends on,
//   KL[b,k] = Qk[b] + Ek[k] + sum_d qa[b,d] T[k,d] + sum_d qb[b,d] T[k,D+d]
//     T[k,d] = psi(se)-psi(ea),  T[k,D+d] = psi(se)-psi(eb)                       (one row of 2D floats per shared row)
//     Ek[k]  = sum_d [lgG(se)-lgG(ea)-lgG(eb)] + ea psi(ea) + eb psi(eb) - se psi(se)
//     Qk[b]  = sum_d lgG(qa)+lgG(qb)-lgG(sq)
// the special functions are evaluated K x D + B x D times instead of B x K x D, and what is left per pair is an
// inner product over 2D features with an operand shared along each axis: a matrix product [B, 2D] x [2D, K], the one
// shape on this path that the matrix cores fit (v_mfma_f32_32x32x2_f32: fp32 operands, fp32 accumulation in a fixed
// order).  The query backward is the other product with the same table,
//   gqa[b,d] = (psi(qa)-psi(sq)) sum_k c[b,k] + sum_k c[b,k] T[k,d]            (c = -upstream gradient; same with b),
// i.e. [B, K] x [K, 2D].  The sums are those of ModelOps<mBetaKL>::fwd / bwd_q taken in another order: the four
// groups are summed separately, which costs some of the tolerance's headroom (measured in the tests), not the bar.
// The entity side of the backward needs no special functions per pair at all (sums of c (e - q), one trigamma
// hook per finished row): it is shared_entity_kernel of smx_shared_impl.h as it stands.
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

// score[b,k] = gamma - (Qk[b] + Ek[k] + sum_j q[b,j] T[k,j]), j over the 2D features ([q1 | q2] against a row of T).
// Both operands have the inner dimension contiguous: a lane reads two neighbouring features per load and feeds
// them to two instructions (instruction t of a group of four features takes feature 4 g + 2 (l / 32) + t).
// Wavefronts 0, 1: the two halves of the q1 part; 2, 3: of the q2 part.
__global__ __launch_bounds__(256) void beta_shared_forward_gemm_kernel(const float* __restrict__ T,
                                                                       const float* __restrict__ Ek,
                                                                       const float* __restrict__ Qk,
                                                                       const float* __restrict__ q1,
                                                                       const float* __restrict__ q2,
                                                                       float* __restrict__ score, int B, int K, int dim,
                                                                       float gamma) {
  __shared__ float part[3 * 16 * 64];
  const int lane = threadIdx.x & 63;
  const int wave = uniform(threadIdx.x >> 6);
  const int tiles_k = (K + 31) / 32;
  const int tile = blockIdx.x;
  const int b0 = (tile / tiles_k) * 32, k0 = (tile % tiles_k) * 32;
  const int half = lane >> 5, col = lane & 31;
  const int my_b = min(b0 + col, B - 1), my_k = min(k0 + col, K - 1);  // rows past the end repeat the last one; never stored
  facc16 acc = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  {
    const int seg = wave >> 1;
    const float2* a = reinterpret_cast<const float2*>((seg ? q2 : q1) + (size_t)my_b * dim) + half;
    const float2* t = reinterpret_cast<const float2*>(T + (size_t)my_k * 2 * dim + (size_t)seg * dim) + half;
    // four groups at a time, the next four requested before these are used (requests past the end repeat the last group)
    const int G = dim / 4;
    const int g_lo = (wave & 1) ? G / 2 : 0, g_hi = (wave & 1) ? G : G / 2;
    float2 av[4], tv[4], an[4], tn[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      av[u] = a[2 * min(g_lo + u, G - 1)];
      tv[u] = t[2 * min(g_lo + u, G - 1)];
    }
    for (int g = g_lo; g < g_hi; g += 4) {
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        an[u] = a[2 * min(g + 4 + u, G - 1)];
        tn[u] = t[2 * min(g + 4 + u, G - 1)];
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        if (g + u < g_hi) {  // uniform
          acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av[u].x, tv[u].x, acc, 0, 0, 0);
          acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av[u].y, tv[u].y, acc, 0, 0, 0);
        }
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        av[u] = an[u];
        tv[u] = tn[u];
      }
    }
  }
  combine_tiles(acc, part, wave, lane);
  const int k = k0 + col;
  if (wave != 0 || k >= K) return;
  const float ek = Ek[k];
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int b = b0 + acc_row(r, lane);
    if (b < B) score[(size_t)b * K + k] = gamma - ((Qk[b] + ek) + acc[r]);
  }
}

// gq[b,n] = kq[b,n] sum_k c[b,k] + sum_k c[b,k] T[k,n], n over the 2D features (n < D: gq1 with kq = psi(qa)-psi(sq),
// else gq2 with psi(qb)-psi(sq)), c = -gscore.  The lanes of a tile's A operand also add up what they load: the
// row sums of c come for free.  Each of the four wavefronts walks a quarter of the list.
__global__ __launch_bounds__(256) void beta_shared_backward_query_gemm_kernel(const float* __restrict__ T,
                                                                              const float* __restrict__ q1,
                                                                              const float* __restrict__ q2,
                                                                              const float* __restrict__ gscore,
                                                                              float* __restrict__ gq1,
                                                                              float* __restrict__ gq2, int B, int K,
                                                                              int dim) {
  __shared__ float part[3 * 16 * 64];
  __shared__ float part_c[3 * 64];
  const int lane = threadIdx.x & 63;
  const int wave = uniform(threadIdx.x >> 6);
  const int tiles_n = (2 * dim + 31) / 32;
  const int tile = blockIdx.x;
  const int b0 = (tile / tiles_n) * 32, n0 = (tile % tiles_n) * 32;
  const int half = lane >> 5, col = lane & 31;
  const int my_b = min(b0 + col, B - 1);
  const int my_n = min(n0 + col, 2 * dim - 1);
  const float* a = gscore + (size_t)my_b * K;
  const float* t = T + my_n;
  facc16 acc = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  float c_sum = 0.f;
  // this wavefront's stretch of the list, a multiple of eight rows: four instructions take eight rows, lanes 0-31
  // supplying rows kk .. kk+3 and lanes 32-63 rows kk+4 .. kk+7 (one 16-byte load of coefficients per lane when the
  // rows of gscore are 16-byte aligned).  The next eight are requested before these are used; a request past the
  // end of the stretch repeats the list's last row with coefficient 0
  const int per = ((K + 31) / 32) * 8;
  const int k_lo = wave * per, k_hi = min(K, k_lo + per);
  const size_t ld = (size_t)2 * dim;
  const bool wide = (K & 3) == 0 && (reinterpret_cast<unsigned long long>(gscore) & 15ull) == 0ull;
  float cv[4], tv[4], cn[4], tn[4];
  auto request = [&](float (&c)[4], float (&tt)[4], int kk0) {
    const int k4 = kk0 + 4 * half;
    if (wide && k4 + 3 < k_hi) {  // (k_hi is a multiple of 4 here: all four rows or none)
      const float4 g = *reinterpret_cast<const float4*>(a + k4);
      c[0] = -g.x;
      c[1] = -g.y;
      c[2] = -g.z;
      c[3] = -g.w;
    } else {
#pragma unroll
      for (int u = 0; u < 4; ++u) c[u] = k4 + u < k_hi ? -a[min(k4 + u, K - 1)] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) tt[u] = t[(size_t)min(k4 + u, K - 1) * ld];
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
    if (b < B && n < 2 * dim) {
      const QBeta q = ModelOps<mBetaKL>::prep_bwd_q(q1[(size_t)b * dim + d], q2[(size_t)b * dim + d]);
      float* out = n < dim ? gq1 : gq2;
      out[(size_t)b * dim + d] = (n < dim ? q.k : q.l) * s + acc[r];
    }
  }
}

// Entity side: ModelOps<mBetaKL>::bwd_e sums c (ea - qa) and c (eb - qb) over the queries, i.e. for list position k
//   S1[k,d] = ea[k,d] C[k] - R[k,d],  S2[k,d] = eb[k,d] C[k] - R[k,D+d],  C[k] = sum_b c[b,k],  R = c^T [K,B] x [q1 | q2] [B,2D]:
// this kernel leaves R [K][2D] and C [K] in the workspace, and shared_entity_kernel turns them into the gradient row
// (the trigamma hook, the clamp mask, the optimizer) as it does with the sums it forms itself.  Both operands
// are read along their contiguous dimension (lane l: c[b + l / 32][k0 + l % 32] and q[b + l / 32][n0 + l % 32]);
// each of the four wavefronts walks a quarter of the queries.
__global__ __launch_bounds__(256) void beta_shared_entity_gemm_kernel(const float* __restrict__ q1,
                                                                      const float* __restrict__ q2,
                                                                      const float* __restrict__ gscore,
                                                                      float* __restrict__ R, float* __restrict__ C, int B,
                                                                      int K, int dim) {
  __shared__ float part[3 * 16 * 64];
  __shared__ float part_c[3 * 64];
  const int lane = threadIdx.x & 63;
  const int wave = uniform(threadIdx.x >> 6);
  const int tiles_n = (2 * dim + 31) / 32;
  const int tile = blockIdx.x;
  const int k0 = (tile / tiles_n) * 32, n0 = (tile % tiles_n) * 32;
  const int half = lane >> 5, col = lane & 31;
  const int my_k = min(k0 + col, K - 1);
  const int my_n = min(n0 + col, 2 * dim - 1);
  const float* a = gscore + my_k;
  const float* t = my_n < dim ? q1 + my_n : q2 + (my_n - dim);
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
      c[u] = b < b_hi ? -a[(size_t)bc * K] : 0.f;
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
  if (n0 == 0 && half == 0 && k0 + col < K) C[k0 + col] = c_sum;
  const int n = n0 + col;
  if (n >= 2 * dim) return;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int k = k0 + acc_row(r, lane);
    if (k < K) R[(size_t)k * 2 * dim + n] = acc[r];
  }
}

// Whether the call can take these kernels: float4-aligned operands and room for T, Ek and Qk in the workspace.
bool beta_shared_fits(size_t dim, const void* table, const void* q1, const void* q2, const void* workspace,
                      size_t workspace_bytes, size_t B, size_t K) {
  if (dim % 4 != 0 || !workspace) return false;
  if (!aligned16(table) || !aligned16(q1) || !aligned16(q2) || !aligned16(workspace)) return false;
  return workspace_bytes >= (K * (2 * dim + 1) + B) * sizeof(float);
}

int beta_shared_forward(hipStream_t st, const float* table, size_t n_rows, const long long* ids, const float* q1,
                        const float* q2, float* score, size_t B, size_t K, size_t dim, const ScoreParams& p, int* err,
                        float* workspace) {
  float* T = workspace;
  float* Ek = T + K * 2 * dim;
  float* Qk = Ek + K;
  hipLaunchKernelGGL(beta_row_terms_kernel<true>, dim3((unsigned)((K + 3) / 4)), dim3(256), 0, st, table, ids, (int)K,
                     (int)dim, (unsigned long long)n_rows, p, T, Ek, err);
  hipLaunchKernelGGL(beta_query_terms_kernel, dim3((unsigned)((B + 3) / 4)), dim3(256), 0, st, q1, q2, (int)B, (int)dim, Qk);
  const size_t tiles = ((B + 31) / 32) * ((K + 31) / 32);
  hipLaunchKernelGGL(beta_shared_forward_gemm_kernel, dim3((unsigned)tiles), dim3(256), 0, st, T, Ek, Qk, q1, q2,
                     score, (int)B, (int)K, (int)dim, p.gamma);
  return check_launch("score forward (shared negatives, beta_kl)");
}

int beta_shared_backward_query(hipStream_t st, const float* table, size_t n_rows, const long long* ids, const float* q1,
                               const float* q2, const float* gscore, float* gq1, float* gq2, size_t B, size_t K,
                               size_t dim, const ScoreParams& p, float* workspace) {
  float* T = workspace;
  hipLaunchKernelGGL(beta_row_terms_kernel<false>, dim3((unsigned)((K + 3) / 4)), dim3(256), 0, st, table, ids, (int)K,
                     (int)dim, (unsigned long long)n_rows, p, T, nullptr, nullptr);
  const size_t tiles = ((B + 31) / 32) * ((2 * dim + 31) / 32);
  hipLaunchKernelGGL(beta_shared_backward_query_gemm_kernel, dim3((unsigned)tiles), dim3(256), 0, st, T, q1, q2,
                     gscore, gq1, gq2, (int)B, (int)K, (int)dim);
  return check_launch("score backward (query, shared negatives, beta_kl)");
}

// R [K][2D] and C [K] for the entity side (see beta_shared_entity_gemm_kernel); workspace: K (2 dim + 1) floats
int beta_shared_entity_sums(hipStream_t st, const float* q1, const float* q2, const float* gscore, size_t B, size_t K,
                            size_t dim, float* workspace) {
  const size_t tiles = ((K + 31) / 32) * ((2 * dim + 31) / 32);
  hipLaunchKernelGGL(beta_shared_entity_gemm_kernel, dim3((unsigned)tiles), dim3(256), 0, st, q1, q2, gscore, workspace,
                     workspace + K * 2 * dim, (int)B, (int)K, (int)dim);
  return check_launch("entity backward (shared negatives, beta_kl sums)");
}

}  // namespace smx
