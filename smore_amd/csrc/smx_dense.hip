// Dense distance operators for any broadcast layout, fp32 and fp64.
//
// These are the layout-general kernels behind smx_dist_forward_* /
// smx_dist_backward_*: entity [be,ne,dim*mul] against query [bc,nc,dim] with
// the modulo broadcast rule of the replaced launch loops
// (smore/common/torchext/common_kernel.h:41-49, 73-81, 108-115).  The
// per-query-negatives layout with 16-byte aligned fp32 rows is routed to the
// vectorised kernels in smx_score.hip instead.
//
// forward : one wavefront per output element, lanes stride the feature axis,
//           xor-butterfly reduction over 64 lanes.
// backward: one workgroup per row of the side being differentiated; each
//           thread owns features d, d+blockDim, ... and walks that row's jobs
//           in ascending job order, so every sum has a fixed order and no
//           atomics are needed.
#include "smx_common.h"
#include "smx_functors.h"

namespace smx {

template <typename T>
__device__ __forceinline__ T wave_sum(T v) {
#pragma unroll
  for (int m = kWave / 2; m > 0; m >>= 1) v += __shfl_xor(v, m, kWave);
  return v;
}

struct Layout {
  size_t bsize, num, be, ne, bc, nc, dim;
};

template <int K, typename T>
__global__ __launch_bounds__(256) void dense_forward_kernel(const T* __restrict__ ent, const T* __restrict__ q1,
                                                            const T* __restrict__ q2, T* __restrict__ dst, Layout L) {
  constexpr int MUL = kind_mul(K);
  const int lane = threadIdx.x & (kWave - 1);
  const size_t waves_per_block = blockDim.x / kWave;
  const size_t total = L.bsize * L.num;
  for (size_t w = blockIdx.x * waves_per_block + threadIdx.x / kWave; w < total; w += (size_t)gridDim.x * waves_per_block) {
    const size_t i = w / L.num, j = w % L.num;
    const T* pe = ent + ((i % L.be) * L.ne + (j % L.ne)) * L.dim * MUL;
    const size_t qrow = ((i % L.bc) * L.nc + (j % L.nc)) * L.dim;
    T s = 0;
    for (size_t d = lane; d < L.dim; d += kWave) {
      const T e1 = pe[d];
      const T e2 = MUL == 2 ? pe[d + L.dim] : (T)0;
      const T a = q1[qrow + d];
      const T b = kind_nq(K) == 2 ? q2[qrow + d] : (T)0;
      s += Term<K, T>::fwd(e1, e2, a, b);
    }
    s = wave_sum(s);
    if (lane == 0) dst[w] = s;
  }
}

// SIDE 0: gradient of the entity rows, SIDE 1: gradient of the query rows.
template <int K, typename T, int SIDE>
__global__ __launch_bounds__(128) void dense_backward_kernel(const T* __restrict__ gout, const T* __restrict__ ent,
                                                             const T* __restrict__ q1, const T* __restrict__ q2,
                                                             T* __restrict__ g_a, T* __restrict__ g_b, Layout L) {
  constexpr int MUL = kind_mul(K);
  constexpr int NQ = kind_nq(K);
  const size_t row = blockIdx.x;
  const size_t own_b = SIDE == 0 ? L.be : L.bc;
  const size_t own_n = SIDE == 0 ? L.ne : L.nc;
  const size_t d0 = row / own_n, d1 = row % own_n;
  const size_t nji = L.bsize / own_b, njj = L.num / own_n;
  for (size_t d = threadIdx.x; d < L.dim; d += blockDim.x) {
    T acc1 = 0, acc2 = 0;
    T own_e1 = 0, own_e2 = 0, own_q1 = 0, own_q2 = 0;
    if (SIDE == 0) {
      own_e1 = ent[row * L.dim * MUL + d];
      if (MUL == 2) own_e2 = ent[row * L.dim * MUL + d + L.dim];
    } else {
      own_q1 = q1[row * L.dim + d];
      if (NQ == 2) own_q2 = q2[row * L.dim + d];
    }
    for (size_t job = 0; job < nji * njj; ++job) {
      const size_t i = (job / njj) * own_b + d0, j = (job % njj) * own_n + d1;
      const T g = gout[i * L.num + j];
      T sink1 = 0, sink2 = 0;
      if (SIDE == 0) {
        const size_t qrow = ((i % L.bc) * L.nc + (j % L.nc)) * L.dim;
        const T a = q1[qrow + d];
        const T b = NQ == 2 ? q2[qrow + d] : (T)0;
        Term<K, T>::bwd(g, own_e1, own_e2, a, b, acc1, acc2, sink1, sink2);
      } else {
        const T* pe = ent + ((i % L.be) * L.ne + (j % L.ne)) * L.dim * MUL;
        const T e1 = pe[d];
        const T e2 = MUL == 2 ? pe[d + L.dim] : (T)0;
        Term<K, T>::bwd(g, e1, e2, own_q1, own_q2, sink1, sink2, acc1, acc2);
      }
    }
    if (SIDE == 0) {
      g_a[row * L.dim * MUL + d] = acc1;
      if (MUL == 2) g_a[row * L.dim * MUL + d + L.dim] = acc2;
    } else {
      g_a[row * L.dim + d] = acc1;
      if (NQ == 2) g_b[row * L.dim + d] = acc2;
    }
  }
}

static int check_layout(const Layout& L) {
  if (L.bsize == 0 || L.num == 0 || L.dim == 0 || L.be == 0 || L.ne == 0 || L.bc == 0 || L.nc == 0)
    return fail(SMX_ERR_SHAPE, "empty dimension in dist layout");
  if (L.bsize % L.be || L.bsize % L.bc || L.num % L.ne || L.num % L.nc)
    return fail(SMX_ERR_SHAPE, "output [%zu,%zu] is not a multiple of entity [%zu,%zu] / query [%zu,%zu]", L.bsize,
                L.num, L.be, L.ne, L.bc, L.nc);
  if (L.be * L.ne > 0x7fffffffull || L.bc * L.nc > 0x7fffffffull)
    return fail(SMX_ERR_SHAPE, "more than 2^31-1 rows on one side");
  return SMX_OK;
}

template <int K, typename T>
static int forward_k(hipStream_t st, const T* ent, const T* q1, const T* q2, T* dst, const Layout& L) {
  const size_t total = L.bsize * L.num;
  size_t blocks = (total + 3) / 4;
  if (blocks > (1u << 20)) blocks = 1u << 20;
  hipLaunchKernelGGL((dense_forward_kernel<K, T>), dim3((unsigned)blocks), dim3(256), 0, st, ent, q1, q2, dst, L);
  return check_launch("dist forward");
}

template <int K, typename T>
static int backward_k(hipStream_t st, const T* gout, const T* ent, const T* q1, const T* q2, T* gent, T* gq1, T* gq2,
                      const Layout& L) {
  hipLaunchKernelGGL((dense_backward_kernel<K, T, 0>), dim3((unsigned)(L.be * L.ne)), dim3(128), 0, st, gout, ent, q1,
                     q2, gent, (T*)nullptr, L);
  hipLaunchKernelGGL((dense_backward_kernel<K, T, 1>), dim3((unsigned)(L.bc * L.nc)), dim3(128), 0, st, gout, ent, q1,
                     q2, gq1, gq2, L);
  return check_launch("dist backward");
}

#define SMX_FOR_EACH_KIND(X) \
  X(kL1) X(kL2) X(kBoxOut) X(kBoxIn) X(kRotate) X(kBetaKL) X(kComplex) X(kDistmult) X(kBetaL2) X(kBetaFisher)

template <typename T>
int dense_forward(int kind, void* stream, const T* ent, const T* q1, const T* q2, T* dst, size_t bsize, size_t num,
                  size_t be, size_t ne, size_t bc, size_t nc, size_t dim) {
  if (kind < 0 || kind >= kNumKinds) return fail(SMX_ERR_KIND, "unknown dist kind %d", kind);
  Layout L{bsize, num, be, ne, bc, nc, dim};
  if (int rc = check_layout(L)) return rc;
  if (!ent || !q1 || !dst || (kind_nq(kind) == 2 && !q2)) return fail(SMX_ERR_ARG, "null tensor pointer");
  hipStream_t st = as_stream(stream);
  switch (kind) {
#define X(KK) \
  case KK:    \
    return forward_k<KK, T>(st, ent, q1, q2, dst, L);
    SMX_FOR_EACH_KIND(X)
#undef X
  }
  return fail(SMX_ERR_KIND, "unknown dist kind %d", kind);
}

template <typename T>
int dense_backward(int kind, void* stream, const T* gout, const T* ent, const T* q1, const T* q2, T* gent, T* gq1,
                   T* gq2, size_t bsize, size_t num, size_t be, size_t ne, size_t bc, size_t nc, size_t dim) {
  if (kind < 0 || kind >= kNumKinds) return fail(SMX_ERR_KIND, "unknown dist kind %d", kind);
  Layout L{bsize, num, be, ne, bc, nc, dim};
  if (int rc = check_layout(L)) return rc;
  if (!gout || !ent || !q1 || !gent || !gq1 || (kind_nq(kind) == 2 && (!q2 || !gq2)))
    return fail(SMX_ERR_ARG, "null tensor pointer");
  hipStream_t st = as_stream(stream);
  switch (kind) {
#define X(KK) \
  case KK:    \
    return backward_k<KK, T>(st, gout, ent, q1, q2, gent, gq1, gq2, L);
    SMX_FOR_EACH_KIND(X)
#undef X
  }
  return fail(SMX_ERR_KIND, "unknown dist kind %d", kind);
}

}  // namespace smx

extern "C" {

int smx_dist_forward_f32(int kind, void* stream, const float* ent, const float* q1, const float* q2, float* dst,
                         size_t bsize, size_t num, size_t be, size_t ne, size_t bc, size_t nc, size_t dim) {
  return smx::dense_forward<float>(kind, stream, ent, q1, q2, dst, bsize, num, be, ne, bc, nc, dim);
}
int smx_dist_forward_f64(int kind, void* stream, const double* ent, const double* q1, const double* q2, double* dst,
                         size_t bsize, size_t num, size_t be, size_t ne, size_t bc, size_t nc, size_t dim) {
  return smx::dense_forward<double>(kind, stream, ent, q1, q2, dst, bsize, num, be, ne, bc, nc, dim);
}
int smx_dist_backward_f32(int kind, void* stream, const float* gout, const float* ent, const float* q1,
                          const float* q2, float* gent, float* gq1, float* gq2, size_t bsize, size_t num, size_t be,
                          size_t ne, size_t bc, size_t nc, size_t dim) {
  return smx::dense_backward<float>(kind, stream, gout, ent, q1, q2, gent, gq1, gq2, bsize, num, be, ne, bc, nc, dim);
}
int smx_dist_backward_f64(int kind, void* stream, const double* gout, const double* ent, const double* q1,
                          const double* q2, double* gent, double* gq1, double* gq2, size_t bsize, size_t num,
                          size_t be, size_t ne, size_t bc, size_t nc, size_t dim) {
  return smx::dense_backward<double>(kind, stream, gout, ent, q1, q2, gent, gq1, gq2, bsize, num, be, ne, bc, nc, dim);
}

}  // extern "C"
