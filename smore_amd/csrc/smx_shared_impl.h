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

template <int M, int VEC, int NIT, int NW, bool REG>
__global__ __launch_bounds__(NW * 64) void shared_entity_kernel(SharedArgs A) {
  constexpr int MUL = model_mul(M);
  constexpr int NQ = model_nq(M);
  constexpr int R = shared_rows_ahead(NIT, NQ);
  extern __shared__ float lds[];  // [NW - 1] partial rows
  const int lane = threadIdx.x & 63;
  const int wave = uniform(threadIdx.x >> 6);
  const int half = A.ncol * VEC;
  const size_t row_len = (size_t)half * MUL;
  const int item = blockIdx.x;
  int m0 = item, m1 = item + 1;
  long long row;
  if (A.by_segment) {
    if (item >= *A.n_uniq) return;  // uniform over the workgroup (ids outside the table form no counted segment)
    m0 = A.seg_start[item];
    m1 = A.seg_start[item + 1];
    row = A.uniq[item];
  } else {
    row = A.ids[item];
    if ((unsigned long long)row >= A.n_rows) row = 0;  // the forward has flagged it; the plan keeps such a row out of every update
  }
  RowRegs<MUL, VEC, NIT> e;
  load_row<MUL, VEC, NIT>(e, A.table + (size_t)row * row_len, half, A.ncol, lane);

  float g1[NIT][VEC], g2[NIT][VEC];
#pragma unroll
  for (int it = 0; it < NIT; ++it)
#pragma unroll
    for (int x = 0; x < VEC; ++x) g1[it][x] = g2[it][x] = 0.f;

  bool have_sums = false;
  if constexpr ((M == mBetaKL || M == mComplex || M == mDistmult) && VEC == 4) {
    if (A.sums_r) {  // uniform: the sums over the queries are there; the first wavefront alone has work
      have_sums = true;
      if (wave == 0) {
        for (int mi = m0; mi < m1; ++mi) {
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
                const float x1 = REG ? reg_apply(e.h[0][it].v[x], A.p) : e.h[0][it].v[x];
                const float x2 = REG ? reg_apply(e.h[MUL - 1][it].v[x], A.p) : e.h[MUL - 1][it].v[x];
                g1[it][x] += x1 * c - r1v[x];
                g2[it][x] += x2 * c - r2v[x];
              } else {                       // the gradient row itself: sum_b g q
                g1[it][x] += r1v[x];
                if (MUL == 2) g2[it][x] += r2v[x];
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
  for (int mi = m0; mi < m1; ++mi) {
    const int k = A.by_segment ? A.order[mi] : mi;
    for (int b0 = b_lo; b0 < b_hi; b0 += 64) {
      const int cnt = min(64, b_hi - b0);
      const size_t mine = (size_t)(b0 + min(lane, cnt - 1)) * A.K + k;
      float my_c0, my_c1;
      ModelOps<M>::coef(A.gscore[mine], A.score[mine], A.p, my_c0, my_c1);
      for (int j0 = 0; j0 < cnt; j0 += R) {
        Pack2<VEC> qa[R][NIT], qb[R][NIT];
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const size_t qoff = (size_t)(b0 + min(j0 + r, cnt - 1)) * half;
#pragma unroll
          for (int it = 0; it < NIT; ++it) {
            const int c = min(lane + 64 * it, A.ncol - 1);
            qa[r][it] = ld<VEC>(A.q1 + qoff, c);
            if constexpr (NQ == 2) qb[r][it] = ld<VEC>(A.q2 + qoff, c);
          }
        }
#pragma unroll
        for (int r = 0; r < R; ++r) {
          if (j0 + r < cnt) {  // uniform
            float c0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(my_c0), j0 + r));
            const float c1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(my_c1), j0 + r));
            if constexpr (M == mL2)
              c0 = l2_pair_coef<VEC, NIT>(c0, A.ncol, lane, [&](int it, int x) { return e.h[0][it].v[x]; },
                                          [&](int it, int x) { return qa[r][it].v[x]; });
#pragma unroll
            for (int it = 0; it < NIT; ++it)
#pragma unroll
              for (int x = 0; x < VEC; ++x) {
                const typename ModelOps<M>::Q q = ModelOps<M>::prep(qa[r][it].v[x], NQ == 2 ? qb[r][it].v[x] : 0.f);
                const float x1 = REG ? reg_apply(e.h[0][it].v[x], A.p) : e.h[0][it].v[x];
                const float x2 = MUL == 2 ? (REG ? reg_apply(e.h[MUL - 1][it].v[x], A.p) : e.h[MUL - 1][it].v[x]) : 0.f;
                ModelOps<M>::bwd_e(c0, c1, x1, x2, q, g1[it][x], g2[it][x]);
              }
          }
        }
      }
    }
  }

  // combine the wavefronts' sums in wavefront order
  auto park = [&](float* buf) {
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      const int c = lane + 64 * it;
      if (c < A.ncol) {
        st<VEC>(buf, c, g1[it]);
        if (MUL == 2) st<VEC>(buf + half, c, g2[it]);
      }
    }
  };
  if (wave > 0) park(lds + (size_t)(wave - 1) * row_len);
  __syncthreads();
  if (wave != 0) return;
  for (int w = 1; w < NW; ++w) {
    RowRegs<MUL, VEC, NIT> o;
    load_row<MUL, VEC, NIT>(o, lds + (size_t)(w - 1) * row_len, half, A.ncol, lane);
#pragma unroll
    for (int it = 0; it < NIT; ++it)
#pragma unroll
      for (int x = 0; x < VEC; ++x) {
        g1[it][x] += o.h[0][it].v[x];
        if (MUL == 2) g2[it][x] += o.h[MUL - 1][it].v[x];
      }
  }
  RowRegs<MUL, VEC, NIT> m0r, v0r;
  if (A.adam_on == kOptAdam) load_row<MUL, VEC, NIT, true>(m0r, A.m + (size_t)row * row_len, half, A.ncol, lane);
  if (A.adam_on && A.adam_on != kOptSgd && !A.squeeze)
    load_row<MUL, VEC, NIT, true>(v0r, A.v + (size_t)row * row_len, half, A.ncol, lane);
  finish_row<M, VEC, NIT, REG>(A, lane, (unsigned)row, item, g1, g2, e, m0r, v0r);
}

template <int M, int VEC, int NIT, bool REG>
int launch_shared_entity_reg(hipStream_t st, const SharedArgs& A) {
  const size_t row_bytes = (size_t)A.ncol * VEC * model_mul(M) * sizeof(float);
  // one workgroup per list position; with a plan the workgroups beyond the number of distinct ids leave at once
  if constexpr ((M == mBetaKL || M == mComplex || M == mDistmult) && VEC == 4) {
    if (A.sums_r) {  // the sums over the queries are there: one wavefront per row finishes it
      hipLaunchKernelGGL((shared_entity_kernel<M, VEC, NIT, 1, REG>), dim3((unsigned)A.K), dim3(64), 0, st, A);
      return check_launch("entity backward (shared negatives, rows from the sums)");
    }
  }
  if (7 * row_bytes <= 60 * 1024)
    hipLaunchKernelGGL((shared_entity_kernel<M, VEC, NIT, 8, REG>), dim3((unsigned)A.K), dim3(8 * 64), 7 * row_bytes, st, A);
  else
    hipLaunchKernelGGL((shared_entity_kernel<M, VEC, NIT, 4, REG>), dim3((unsigned)A.K), dim3(4 * 64), 3 * row_bytes, st, A);
  return check_launch("entity backward (shared negatives)");
}

template <int M, int VEC, int NIT>
int launch_shared_entity(hipStream_t st, const SharedArgs& A) {
  if constexpr (M == mBetaKL) {
    if (A.p.reg_on) return launch_shared_entity_reg<M, VEC, NIT, true>(st, A);
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
