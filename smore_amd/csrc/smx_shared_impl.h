// Entity-side backward for negatives that every query of the batch shares.
//
// SMORE's training scripts all run with --share_negative: the sampler draws ONE list of K negative ids per
// batch (smore/cpp_sampler/online_sampler.py:155-157), the model code looks those K rows up once and scores
// them against every query ([1,K,row] against [B,1,D], smore/models/kg_reasoning.py:349-355), and a mask
// removes the pairs that are true answers (is_negative_mat, smore/training/train_process.py:195-196; it
// reaches this kernel folded into the upstream gradient).  The gradient of shared row k is then a sum over
// all B queries,
//     g[k,:] = sum_b  d(gscore[b,k] * score[b,k]) / d row,
// which the reference forms with dist_backward_ent_kernel (smore/common/torchext/common_kernel.h:59-89) and
// merges and applies with embed_optimizer.py:39-48, 208-252.
//
// Here one workgroup owns one shared row (or, given a segment plan over the K ids, one distinct id and all
// the list positions that hold it): the row stays in registers, the wavefronts split the queries into
// contiguous stretches and stream them, the partial sums are combined through LDS in wavefront order (fixed
// summation order, no float atomics), and the first wavefront finishes the row -- the model's hook, the clamp
// mask, then either the gradient row itself (for a step that merges it with other index streams) or the
// optimizer update of w, m, v in place.
#pragma once
#include "smx_common.h"
#include "smx_models.h"
#include "smx_rowupdate.h"
#include "smx_wave.h"

namespace smx {

struct SharedArgs : RowSink {
  const long long* ids;  // [K] the shared entity ids
  const float* q1;
  const float* q2;
  const float* score;   // [B, K]
  const float* gscore;  // [B, K]
  int B, K;
  unsigned long long n_rows;
  // by_segment: one workgroup per distinct id of a segment plan built over the K ids (and nothing else);
  // finished rows go where the sink says (merged row number = segment number).
  // else: one workgroup per list position k; its row of the sink's `merged` is row k.
  int by_segment;
  const int* order;
  const int* seg_start;
  const long long* uniq;
  const int* n_uniq;
  // beta_kl, complex, distmult: the sums over the queries come from a matrix product (R [K][nq dim] and, beta_kl,
  // C [K], see smx_shared_gemm.hip) instead of being formed here
  const float* sums_r;
  const float* sums_c;
};

// queries whose rows a wavefront requests before it uses the first
constexpr int shared_rows_ahead(int nit, int nq) { return nit * nq <= 2 ? 4 : (nit * nq <= 4 ? 2 : 1); }

// RW: rows per workgroup.  With two, every query row a wavefront fetches meets both of them: half the requests
// to the L2 per pair, which is what bounds this kernel once the B x K pairs are many (B = 512, K = 1024, 400-float
// box rows: 1.7 GB of query rows through the L2 in 76 us with one row per workgroup, 62 us with two; rotate rows of
// 800 floats: 105 -> 89 us).  A row's sum has the same
// terms in the same order for either value.
template <int M, int VEC, int NIT, int NW, bool REG, int RW>
__global__ __launch_bounds__(NW * 64) void shared_entity_kernel(SharedArgs A) {
  constexpr int MUL = model_mul(M);
  constexpr int NQ = model_nq(M);
  constexpr int R = RW > 1 ? 2 : shared_rows_ahead(NIT, NQ);
  extern __shared__ float lds[];  // [NW - 1][RW] partial rows
  const int lane = threadIdx.x & 63;
  const int wave = uniform(threadIdx.x >> 6);
  const int half = A.ncol * VEC;
  const size_t row_len = (size_t)half * MUL;
  const int item0 = blockIdx.x * RW;
  const int n_items = A.by_segment ? *A.n_uniq : A.K;  // (ids outside the table form no counted segment)
  if (item0 >= n_items) return;                         // uniform over the workgroup
  int m0[RW], len[RW];
  long long row[RW];
  int steps = 0;
#pragma unroll
  for (int r = 0; r < RW; ++r) {
    const int item = item0 + r;
    if (item >= n_items) {  // no such row: an empty list, and nothing is finished for it
      m0[r] = 0;
      len[r] = 0;
      row[r] = row[0];
    } else if (A.by_segment) {
      m0[r] = A.seg_start[item];
      len[r] = A.seg_start[item + 1] - m0[r];
      row[r] = A.uniq[item];
    } else {
      m0[r] = item;
      len[r] = 1;
      row[r] = A.ids[item];
      if ((unsigned long long)row[r] >= A.n_rows) row[r] = 0;  // the forward has flagged it; the plan keeps such a row out of every update
    }
    steps = max(steps, len[r]);
  }
  RowRegs<MUL, VEC, NIT> e[RW];
#pragma unroll
  for (int r = 0; r < RW; ++r) load_row<MUL, VEC, NIT>(e[r], A.table + (size_t)row[r] * row_len, half, A.ncol, lane);

  float g1[RW][NIT][VEC], g2[RW][NIT][VEC];
#pragma unroll
  for (int r = 0; r < RW; ++r)
#pragma unroll
    for (int it = 0; it < NIT; ++it)
#pragma unroll
      for (int x = 0; x < VEC; ++x) g1[r][it][x] = g2[r][it][x] = 0.f;

  bool have_sums = false;
  if constexpr ((M == mBetaKL || M == mComplex || M == mDistmult) && VEC == 4 && RW == 1) {
    if (A.sums_r) {  // uniform: the sums over the queries are there; the first wavefront alone has work
      have_sums = true;
      if (wave == 0) {
        for (int mi = m0[0]; mi < m0[0] + len[0]; ++mi) {
          const int k = A.by_segment ? A.order[mi] : mi;
          const float4* r = reinterpret_cast<const float4*>(A.sums_r + (size_t)k * NQ * half);
          const float c = M == mBetaKL ? A.sums_c[k] : 0.f;
#pragma unroll
          for (int it = 0; it < NIT; ++it) {
            const int col = min(lane + 64 * it, A.ncol - 1);
            const float4 r1 = r[col], r2 = NQ == 2 ? r[A.ncol + col] : r1;
            const float r1v[4] = {r1.x, r1.y, r1.z, r1.w}, r2v[4] = {r2.x, r2.y, r2.z, r2.w};
#pragma unroll
            for (int x = 0; x < VEC; ++x) {
              if constexpr (M == mBetaKL) {  // S1 = ea C - R, S2 = eb C - R'
                const float x1 = REG ? reg_apply(e[0].h[0][it].v[x], A.p) : e[0].h[0][it].v[x];
                const float x2 = REG ? reg_apply(e[0].h[MUL - 1][it].v[x], A.p) : e[0].h[MUL - 1][it].v[x];
                g1[0][it][x] += x1 * c - r1v[x];
                g2[0][it][x] += x2 * c - r2v[x];
              } else {                       // the gradient row itself: sum_b g q
                g1[0][it][x] += r1v[x];
                if (MUL == 2) g2[0][it][x] += r2v[x];
              }
            }
          }
        }
      }
    }
  }
  // this wavefront's stretch of the queries
  const int per_wave = (A.B + NW - 1) / NW;
  const int b_lo = have_sums ? 0 : wave * per_wave;
  const int b_hi = have_sums ? 0 : min(A.B, b_lo + per_wave);
  for (int s = 0; s < steps; ++s) {  // the s-th list position of every row (a row's positions in list order)
    int k[RW];
#pragma unroll
    for (int r = 0; r < RW; ++r) k[r] = s < len[r] ? (A.by_segment ? A.order[m0[r] + s] : m0[r] + s) : -1;
    for (int b0 = b_lo; b0 < b_hi; b0 += 64) {
      const int cnt = min(64, b_hi - b0);
      float my_c0[RW], my_c1[RW];
#pragma unroll
      for (int r = 0; r < RW; ++r) {
        const size_t mine = (size_t)(b0 + min(lane, cnt - 1)) * A.K + max(k[r], 0);
        ModelOps<M>::coef(A.gscore[mine], A.score[mine], A.p, my_c0[r], my_c1[r]);
      }
      for (int j0 = 0; j0 < cnt; j0 += R) {
        Pack2<VEC> qa[R][NIT], qb[R][NIT];
#pragma unroll
        for (int u = 0; u < R; ++u) {
          const size_t qoff = (size_t)(b0 + min(j0 + u, cnt - 1)) * half;
#pragma unroll
          for (int it = 0; it < NIT; ++it) {
            const int c = min(lane + 64 * it, A.ncol - 1);
            qa[u][it] = ld<VEC>(A.q1 + qoff, c);
            if constexpr (NQ == 2) qb[u][it] = ld<VEC>(A.q2 + qoff, c);
          }
        }
#pragma unroll
        for (int u = 0; u < R; ++u) {
          if (j0 + u < cnt) {  // uniform
#pragma unroll
            for (int r = 0; r < RW; ++r) {
              if (k[r] < 0) continue;  // uniform
              float c0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(my_c0[r]), j0 + u));
              const float c1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(my_c1[r]), j0 + u));
              if constexpr (M == mL2)
                c0 = l2_pair_coef<VEC, NIT>(c0, A.ncol, lane, [&](int it, int x) { return e[r].h[0][it].v[x]; },
                                            [&](int it, int x) { return qa[u][it].v[x]; });
#pragma unroll
              for (int it = 0; it < NIT; ++it)
#pragma unroll
                for (int x = 0; x < VEC; ++x) {
                  const typename ModelOps<M>::Q q = ModelOps<M>::prep(qa[u][it].v[x], NQ == 2 ? qb[u][it].v[x] : 0.f);
                  const float x1 = REG ? reg_apply(e[r].h[0][it].v[x], A.p) : e[r].h[0][it].v[x];
                  const float x2 =
                      MUL == 2 ? (REG ? reg_apply(e[r].h[MUL - 1][it].v[x], A.p) : e[r].h[MUL - 1][it].v[x]) : 0.f;
                  ModelOps<M>::bwd_e(c0, c1, x1, x2, q, g1[r][it][x], g2[r][it][x]);
                }
            }
          }
        }
      }
    }
  }

  // combine the wavefronts' sums in wavefront order
  if (wave > 0) {
#pragma unroll
    for (int r = 0; r < RW; ++r) {
      float* buf = lds + ((size_t)(wave - 1) * RW + r) * row_len;
#pragma unroll
      for (int it = 0; it < NIT; ++it) {
        const int c = lane + 64 * it;
        if (c < A.ncol) {
          st<VEC>(buf, c, g1[r][it]);
          if (MUL == 2) st<VEC>(buf + half, c, g2[r][it]);
        }
      }
    }
  }
  __syncthreads();
  if (wave != 0) return;
#pragma unroll
  for (int r = 0; r < RW; ++r) {
    if (item0 + r >= n_items) break;  // uniform
    for (int w = 1; w < NW; ++w) {
      RowRegs<MUL, VEC, NIT> o;
      load_row<MUL, VEC, NIT>(o, lds + ((size_t)(w - 1) * RW + r) * row_len, half, A.ncol, lane);
#pragma unroll
      for (int it = 0; it < NIT; ++it)
#pragma unroll
        for (int x = 0; x < VEC; ++x) {
          g1[r][it][x] += o.h[0][it].v[x];
          if (MUL == 2) g2[r][it][x] += o.h[MUL - 1][it].v[x];
        }
    }
    RowRegs<MUL, VEC, NIT> m0r, v0r;
    if (A.adam_on == kOptAdam) load_row<MUL, VEC, NIT, true>(m0r, A.m + (size_t)row[r] * row_len, half, A.ncol, lane);
    if (A.adam_on && A.adam_on != kOptSgd && !A.squeeze)
      load_row<MUL, VEC, NIT, true>(v0r, A.v + (size_t)row[r] * row_len, half, A.ncol, lane);
    finish_row<M, VEC, NIT, REG>(A, lane, (unsigned)row[r], item0 + r, g1[r], g2[r], e[r], m0r, v0r);
  }
}

template <int M, int VEC, int NIT, bool REG>
int launch_shared_entity_reg(hipStream_t st, const SharedArgs& A) {
  const size_t row_bytes = (size_t)A.ncol * VEC * model_mul(M) * sizeof(float);
  // one workgroup per list position (or two); with a plan the workgroups beyond the number of distinct ids leave at once
  if constexpr ((M == mBetaKL || M == mComplex || M == mDistmult) && VEC == 4) {
    if (A.sums_r) {  // the sums over the queries are there: one wavefront per row finishes it
      hipLaunchKernelGGL((shared_entity_kernel<M, VEC, NIT, 1, REG, 1>), dim3((unsigned)A.K), dim3(64), 0, st, A);
      return check_launch("entity backward (shared negatives, rows from the sums)");
    }
  }
  // two rows per workgroup where their registers fit beside the queries in flight and enough workgroups remain
  // (not BetaE, whose special-function terms need the registers: it spills with two rows; its shared lists are
  // matrix products anyway)
  if constexpr (VEC == 4 && NIT * model_mul(M) <= 4 && M != mBetaKL) {
    if (A.K >= 512 && A.B >= 64 && 14 * row_bytes <= 60 * 1024) {
      hipLaunchKernelGGL((shared_entity_kernel<M, VEC, NIT, 8, REG, 2>), dim3((unsigned)((A.K + 1) / 2)), dim3(8 * 64),
                         14 * row_bytes, st, A);
      return check_launch("entity backward (shared negatives, two rows per workgroup)");
    }
  }
  if (7 * row_bytes <= 60 * 1024)
    hipLaunchKernelGGL((shared_entity_kernel<M, VEC, NIT, 8, REG, 1>), dim3((unsigned)A.K), dim3(8 * 64), 7 * row_bytes, st, A);
  else
    hipLaunchKernelGGL((shared_entity_kernel<M, VEC, NIT, 4, REG, 1>), dim3((unsigned)A.K), dim3(4 * 64), 3 * row_bytes, st, A);
  return check_launch("entity backward (shared negatives)");
}

template <int M, int VEC, int NIT>
int launch_shared_entity(hipStream_t st, const SharedArgs& A) {
  if constexpr (M == mBetaKL || M == mComplex || M == mDistmult) {
    if (M == mBetaKL ? A.p.reg_on : A.p.norm_on) return launch_shared_entity_reg<M, VEC, NIT, true>(st, A);
  }
  return launch_shared_entity_reg<M, VEC, NIT, false>(st, A);
}

// Instantiated once per model in its own translation unit (smx_shared_inst_*.hip).
template <int M>
int shared_entity_dispatch(hipStream_t st, const SharedArgs& A, int vec, int nit) {
  if (vec == 4) {
    switch (nit) {
      case 1: return launch_shared_entity<M, 4, 1>(st, A);
      case 2: return launch_shared_entity<M, 4, 2>(st, A);
      case 4: return launch_shared_entity<M, 4, 4>(st, A);
      default: return launch_shared_entity<M, 4, 8>(st, A);
    }
  }
  switch (nit) {
    case 1: return launch_shared_entity<M, 1, 1>(st, A);
    case 2: return launch_shared_entity<M, 1, 2>(st, A);
    default: return launch_shared_entity<M, 1, 4>(st, A);
  }
}

}  // namespace smx
