// Forward for negatives that every query of the batch shares (--share_negative: one list of K ids per batch,
// smore/cpp_sampler/online_sampler.py:155-157; scored as [1,K,row] against [B,1,D], smore/models/kg_reasoning.py:349-355).
//
// The K rows meet all B queries, so a workgroup fetches a few of them once, stages them in LDS, and each of its
// eight wavefronts -- one query each, kept in registers -- scores that query against all of them: a row costs one
// trip from the L2 per eight queries instead of one per query, and the row loop reads LDS.  A thread's share of
// the next tile is requested into registers before the current tile is used.  Per pair the arithmetic is that
// of score_forward_kernel (same accumulation per lane, same reduction), so scores are the same bits.
//
// For l1, l2, box and rotate (the inner-product models and BetaE are matrix products for a shared list,
// smx_shared_gemm.hip) and rows of 16-byte aligned float4 columns, up to 128 columns per half (two per lane);
// other shapes use the id-driven kernels with the shared list.
#pragma once
#include "smx_common.h"
#include "smx_models.h"
#include "smx_wave.h"

namespace smx {

struct SharedFwdArgs {
  const float* table;
  const long long* ids;  // [K]
  const float* q1;
  const float* q2;
  float* score;          // [B, K]
  int B, K, ncol;        // ncol float4 columns per half row
  unsigned long long n_rows;
  ScoreParams p;
  int* err;
};

constexpr int kSfWaves = 8;                       // queries per workgroup, one per wavefront
constexpr int kSfThreads = kSfWaves * 64;
constexpr int kSfChunk = 64;                      // shared rows per workgroup
constexpr int kSfPer = 2;                         // float4 pieces of a tile per thread
constexpr int kSfTile4 = kSfThreads * kSfPer;     // a tile: 1024 float4 = 16 KiB of rows

typedef float sfvec4 __attribute__((ext_vector_type(4)));

// grid (ceil(B / 8), ceil(K / 64)); LDS: 64 row offsets + one tile
template <int M, int NIT>
__global__ __launch_bounds__(kSfThreads) void shared_forward_kernel(SharedFwdArgs A) {
  constexpr int MUL = model_mul(M);
  constexpr int NQ = model_nq(M);
  __shared__ unsigned long long row_off[kSfChunk];
  __shared__ __align__(16) sfvec4 tile[kSfTile4];
  const int lane = threadIdx.x & 63;
  const int wave = uniform(threadIdx.x >> 6);
  const int ncol = A.ncol, dim = ncol * 4;
  const int rl4 = ncol * MUL;                     // float4 pieces per row
  const int tile_rows = kSfTile4 / rl4;           // >= 4: rl4 <= 256
  const int b_raw = blockIdx.x * kSfWaves + wave;
  const int b = min(b_raw, A.B - 1);              // a wavefront past the last query computes along (barriers)
  const int k0 = blockIdx.y * kSfChunk, k1 = min(A.K, k0 + kSfChunk);

  if (threadIdx.x < kSfChunk) {
    long long row = A.ids[min(k0 + (int)threadIdx.x, k1 - 1)];
    if ((unsigned long long)row >= A.n_rows) {    // remember it, read row 0 instead (as every scorer of the library does)
      if (A.err) *A.err = 1;
      row = 0;
    }
    row_off[threadIdx.x] = (unsigned long long)row * (unsigned long long)(rl4 * 4);
  }
  typename ModelOps<M>::Q q[NIT][4];
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    const int c = min(lane + 64 * it, ncol - 1);  // lanes past the row end hold a copy of the last column
#pragma unroll
    for (int v = 0; v < 4; ++v)
      q[it][v] = prep_forward<M>(A.q1[(size_t)b * dim + c * 4 + v], NQ == 2 ? A.q2[(size_t)b * dim + c * 4 + v] : 0.f);
  }
  __syncthreads();

  // which piece of a tile this thread carries: the same for every tile
  int pr[kSfPer], pc[kSfPer];
#pragma unroll
  for (int u = 0; u < kSfPer; ++u) {
    const int i = threadIdx.x + u * kSfThreads;
    pr[u] = i / rl4;
    pc[u] = i - pr[u] * rl4;
  }
  sfvec4 next[kSfPer];
  auto request = [&](int kt) {
    const int rows_here = min(tile_rows, k1 - kt);
#pragma unroll
    for (int u = 0; u < kSfPer; ++u)
      if (pr[u] < rows_here) next[u] = reinterpret_cast<const sfvec4*>(A.table + row_off[kt - k0 + pr[u]])[pc[u]];
  };
  request(k0);
  for (int kt = k0; kt < k1; kt += tile_rows) {
    const int rows_here = min(tile_rows, k1 - kt);
    __syncthreads();  // the previous rows have been used by every wavefront
#pragma unroll
    for (int u = 0; u < kSfPer; ++u)
      if (pr[u] < rows_here) tile[threadIdx.x + u * kSfThreads] = next[u];
    __syncthreads();
    if (kt + tile_rows < k1) request(kt + tile_rows);
    for (int r = 0; r < rows_here; ++r) {
      const sfvec4* t = tile + r * rl4;
      float mine = 0.f;
#pragma unroll
      for (int it = 0; it < NIT; ++it) {
        const int c = min(lane + 64 * it, ncol - 1);
        const sfvec4 e1 = t[c];
        sfvec4 e2 = e1;
        if constexpr (MUL == 2) e2 = t[ncol + c];
        float a0 = 0.f, a1 = 0.f;
#pragma unroll
        for (int v = 0; v < 4; ++v) ModelOps<M>::fwd(e1[v], MUL == 2 ? e2[v] : 0.f, q[it][v], a0, a1);
        const float f = ModelOps<M>::fold(a0, a1, A.p);
        mine += lane + 64 * it < ncol ? f : 0.f;
      }
      const float folded = wave_sum_last_f32(mine);
      if (lane == 63 && b_raw < A.B) A.score[(size_t)b * A.K + kt + r] = ModelOps<M>::score(folded, A.p);
    }
  }
}

// Instantiated once per model in its own translation unit (smx_shared_inst_*.hip).
template <int M>
int shared_forward_dispatch(hipStream_t st, const SharedFwdArgs& A, int nit) {
  const dim3 grid((unsigned)((A.B + kSfWaves - 1) / kSfWaves), (unsigned)((A.K + kSfChunk - 1) / kSfChunk));
  if (nit == 1)
    hipLaunchKernelGGL((shared_forward_kernel<M, 1>), grid, dim3(kSfThreads), 0, st, A);
  else
    hipLaunchKernelGGL((shared_forward_kernel<M, 2>), grid, dim3(kSfThreads), 0, st, A);
  return check_launch("score forward (shared negatives)");
}

// Whether a call has the shape these kernels are written for.
inline bool shared_forward_fits(int model, int vec, int nit) {
  return (model == mL1 || model == mL2 || model == mBox || model == mRotate) && vec == 4 && nit <= 2;
}

}  // namespace smx
