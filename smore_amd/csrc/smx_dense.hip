// Dense distance operators for any broadcast layout, fp32 and fp64.
//
// These are the layout-general kernels behind smx_dist_forward_* /
// smx_dist_backward_*: entity [be,ne,dim*mul] against query [bc,nc,dim] with
// the modulo broadcast rule of the replaced launch loops
// (smore/common/torchext/common_kernel.h:41-49, 73-81, 108-115).
//
// General kernels (any layout, fp32 and fp64):
// forward : one wavefront per output element, lanes stride the feature axis,
//           xor-butterfly reduction over 64 lanes.
// backward: one workgroup per row of the side being differentiated; each
//           thread owns features d, d+blockDim, ... and walks that row's jobs
//           in ascending job order, so every sum has a fixed order and no
//           atomics are needed.
//
// Per-query kernels (fp32, 16-byte aligned rows, entity [B,N,dim*mul] against query [B,1,dim]: the
// layout of the models' negatives [B,K] and positives [B,1], kg_reasoning.py:342-355): the query lives
// in LDS / registers, every entity row is read once with 16-byte loads, and the backward writes the
// row gradient and accumulates the query gradient in the same pass.  Shared negatives [1,N,.] and the
// reverse layout (entity [B,1,.] against query [B,N,.]) have kernels of the same build.
#include <type_traits>

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

// ---- per-query layout, fp32 -------------------------------------------------------------------
typedef float dvec4 __attribute__((ext_vector_type(4)));
constexpr int kPqBwdWaves = 8;

template <int K>
__device__ __forceinline__ float pq_row_terms(const dvec4* __restrict__ pe, const float* lds, int ncol, int dim, int lane) {
  constexpr int MUL = kind_mul(K), NQ = kind_nq(K);
  float s = 0.f;
  for (int c = lane; c < ncol; c += kWave) {
    const dvec4 e1 = pe[c];
    const dvec4 e2 = MUL == 2 ? pe[c + ncol] : dvec4{0.f, 0.f, 0.f, 0.f};
    const dvec4 a = reinterpret_cast<const dvec4*>(lds)[c];
    const dvec4 b = NQ == 2 ? reinterpret_cast<const dvec4*>(lds + dim)[c] : dvec4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int x = 0; x < 4; ++x) s += Term<K, float>::fwd(e1[x], e2[x], a[x], b[x]);
  }
  return s;
}

// One workgroup per (query, tile of rows); its four wavefronts take the tile's rows two at a time.
template <int K, bool SHARED = false>
__global__ __launch_bounds__(256) void dense_pq_forward_kernel(const float* __restrict__ ent, const float* __restrict__ q1,
                                                               const float* __restrict__ q2, float* __restrict__ dst,
                                                               int num, int dim, int tiles, int rows_per_tile) {
  constexpr int MUL = kind_mul(K), NQ = kind_nq(K);
  extern __shared__ float lds[];  // q1[dim] | q2[dim]
  const int b = blockIdx.x / tiles, tile = blockIdx.x - b * tiles;
  for (int d = threadIdx.x; d < dim; d += 256) {
    lds[d] = q1[(size_t)b * dim + d];
    if (NQ == 2) lds[dim + d] = q2[(size_t)b * dim + d];
  }
  __syncthreads();
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int ncol = dim / 4;
  const int k1 = min(num, (tile + 1) * rows_per_tile);
  const size_t row_len = (size_t)dim * MUL;
  for (int k = tile * rows_per_tile + wave; k < k1; k += 8) {
    const size_t r0 = (size_t)b * num + k;
    const bool two = k + 4 < k1;
    const size_t r1 = two ? r0 + 4 : r0;
    const size_t e0 = SHARED ? (size_t)k : r0, e1 = SHARED ? (size_t)(two ? k + 4 : k) : r1;  // entity rows
    float s0 = pq_row_terms<K>(reinterpret_cast<const dvec4*>(ent + e0 * row_len), lds, ncol, dim, lane);
    float s1 = pq_row_terms<K>(reinterpret_cast<const dvec4*>(ent + e1 * row_len), lds, ncol, dim, lane);
    s0 = wave_sum(s0);
    s1 = wave_sum(s1);
    if (lane == 0) {
      dst[r0] = s0;
      if (two) dst[r1] = s1;
    }
  }
}

// One workgroup of eight wavefronts per query.  Lane l owns the 16-byte columns l, l+64, ... of the row
// (NIT of them); wavefront w takes rows w, w+8, ...  For every row it writes the row's gradient and adds
// the row's contribution to its query-gradient registers; the eight partial query gradients are summed
// through LDS in wavefront order, so the result does not depend on timing.
// SHARED: the entity rows are the same [1,N,.] for every query (--share_negative, online_sampler.py:155-157);
// this kernel then gives the query gradients only, and dense_shared_entity_backward_kernel the rows'.
template <int K, int NIT, bool SHARED = false>
__global__ __launch_bounds__(kPqBwdWaves * kWave) void dense_pq_backward_kernel(
    const float* __restrict__ gout, const float* __restrict__ ent, const float* __restrict__ q1,
    const float* __restrict__ q2, float* __restrict__ gent, float* __restrict__ gq1, float* __restrict__ gq2, int num,
    int dim) {
  constexpr int MUL = kind_mul(K), NQ = kind_nq(K);
  extern __shared__ float lds[];  // [waves][NQ][dim]
  const int b = blockIdx.x;
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int ncol = dim / 4;
  const size_t row_len = (size_t)dim * MUL;
  const dvec4 zero = {0.f, 0.f, 0.f, 0.f};
  dvec4 qa[NIT], qb[NIT], acc1[NIT], acc2[NIT];
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    const int c = min(lane + kWave * it, ncol - 1);
    qa[it] = reinterpret_cast<const dvec4*>(q1 + (size_t)b * dim)[c];
    qb[it] = NQ == 2 ? reinterpret_cast<const dvec4*>(q2 + (size_t)b * dim)[c] : zero;
    acc1[it] = acc2[it] = zero;
  }
  for (int k = wave; k < num; k += kPqBwdWaves) {
    const size_t r = (size_t)b * num + k;
    const float g = gout[r];
    const size_t er = SHARED ? (size_t)k : r;
    const dvec4* pe = reinterpret_cast<const dvec4*>(ent + er * row_len);
    dvec4* pg = reinterpret_cast<dvec4*>(gent + er * row_len);
    dvec4 e1[NIT], e2[NIT];
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      const int c = min(lane + kWave * it, ncol - 1);
      e1[it] = pe[c];
      e2[it] = MUL == 2 ? pe[c + ncol] : zero;
    }
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      const int c = lane + kWave * it;
      if (c < ncol) {
        dvec4 ge1 = zero, ge2 = zero;
#pragma unroll
        for (int x = 0; x < 4; ++x) {
          float a1 = 0.f, a2 = 0.f, b1 = acc1[it][x], b2 = acc2[it][x];
          Term<K, float>::bwd(g, e1[it][x], e2[it][x], qa[it][x], qb[it][x], a1, a2, b1, b2);
          ge1[x] = a1;
          ge2[x] = a2;
          acc1[it][x] = b1;
          acc2[it][x] = b2;
        }
        if (!SHARED) {
          __builtin_nontemporal_store(ge1, pg + c);
          if (MUL == 2) __builtin_nontemporal_store(ge2, pg + c + ncol);
        }
      }
    }
  }
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    const int c = lane + kWave * it;
    if (c < ncol) {
      reinterpret_cast<dvec4*>(lds + (size_t)(wave * NQ + 0) * dim)[c] = acc1[it];
      if (NQ == 2) reinterpret_cast<dvec4*>(lds + (size_t)(wave * NQ + 1) * dim)[c] = acc2[it];
    }
  }
  __syncthreads();
  for (int d = threadIdx.x; d < dim; d += kPqBwdWaves * kWave) {
    float s1 = 0.f, s2 = 0.f;
#pragma unroll
    for (int w = 0; w < kPqBwdWaves; ++w) {
      s1 += lds[(size_t)(w * NQ + 0) * dim + d];
      if (NQ == 2) s2 += lds[(size_t)(w * NQ + 1) * dim + d];
    }
    gq1[(size_t)b * dim + d] = s1;
    if (NQ == 2) gq2[(size_t)b * dim + d] = s2;
  }
}

// Shared entity rows: gradient of row j = sum over the queries i of gout[i,j] * d term / d e.  One
// workgroup per row, the row in registers; wavefront w takes queries w, w+8, ... in ascending order and
// the eight partial sums are combined through LDS in wavefront order.
template <int K, int NIT>
__global__ __launch_bounds__(kPqBwdWaves * kWave) void dense_shared_entity_backward_kernel(
    const float* __restrict__ gout, const float* __restrict__ ent, const float* __restrict__ q1,
    const float* __restrict__ q2, float* __restrict__ gent, int bsize, int num, int dim) {
  constexpr int MUL = kind_mul(K), NQ = kind_nq(K);
  extern __shared__ float lds[];  // [waves][MUL][dim]
  const int j = blockIdx.x;
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int ncol = dim / 4;
  const size_t row_len = (size_t)dim * MUL;
  const dvec4 zero = {0.f, 0.f, 0.f, 0.f};
  dvec4 e1[NIT], e2[NIT], acc1[NIT], acc2[NIT];
  const dvec4* pe = reinterpret_cast<const dvec4*>(ent + (size_t)j * row_len);
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    const int c = min(lane + kWave * it, ncol - 1);
    e1[it] = pe[c];
    e2[it] = MUL == 2 ? pe[c + ncol] : zero;
    acc1[it] = acc2[it] = zero;
  }
  for (int i = wave; i < bsize; i += kPqBwdWaves) {
    const float g = gout[(size_t)i * num + j];
    const dvec4* pa = reinterpret_cast<const dvec4*>(q1 + (size_t)i * dim);
    const dvec4* pb = reinterpret_cast<const dvec4*>(q2 + (size_t)i * dim);
    dvec4 qa[NIT], qb[NIT];
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      const int c = min(lane + kWave * it, ncol - 1);
      qa[it] = pa[c];
      qb[it] = NQ == 2 ? pb[c] : zero;
    }
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        float a1 = acc1[it][x], a2 = acc2[it][x], s1 = 0.f, s2 = 0.f;
        Term<K, float>::bwd(g, e1[it][x], e2[it][x], qa[it][x], qb[it][x], a1, a2, s1, s2);
        acc1[it][x] = a1;
        acc2[it][x] = a2;
      }
    }
  }
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    const int c = lane + kWave * it;
    if (c < ncol) {
      reinterpret_cast<dvec4*>(lds + (size_t)(wave * MUL + 0) * dim)[c] = acc1[it];
      if (MUL == 2) reinterpret_cast<dvec4*>(lds + (size_t)(wave * MUL + 1) * dim)[c] = acc2[it];
    }
  }
  __syncthreads();
  for (int d = threadIdx.x; d < dim * MUL; d += kPqBwdWaves * kWave) {
    const int h = d / dim, dd = d - h * dim;
    float sum = 0.f;
#pragma unroll
    for (int w = 0; w < kPqBwdWaves; ++w) sum += lds[(size_t)(w * MUL + h) * dim + dd];
    gent[(size_t)j * row_len + d] = sum;
  }
}

// entity [1,N,.] shared by the queries [B,1,.]
static bool shared_layout(const Layout& L, const void* a, const void* b, const void* c, const void* d, const void* e,
                          const void* f, const void* g) {
  if (L.be != 1 || L.bc != L.bsize || L.ne != L.num || L.nc != 1 || L.bsize < 2) return false;
  if (L.dim % 4 != 0 || L.dim > 1024 || L.bsize * L.num > 0x7fffffffull) return false;
  return aligned16(a) && aligned16(b) && aligned16(c) && aligned16(d) && aligned16(e) && aligned16(f) && aligned16(g);
}

template <int K>
static int backward_shared(hipStream_t st, const float* gout, const float* ent, const float* q1, const float* q2,
                           float* gent, float* gq1, float* gq2, const Layout& L) {
  const dim3 block(kPqBwdWaves * kWave);
  const int num = (int)L.num, dim = (int)L.dim, bsize = (int)L.bsize;
  const size_t ncol = L.dim / 4;
  const size_t lds_q = (size_t)kPqBwdWaves * kind_nq(K) * L.dim * sizeof(float);
  const size_t lds_e = (size_t)kPqBwdWaves * kind_mul(K) * L.dim * sizeof(float);
#define SMX_SHARED_LAUNCH(NIT_)                                                                                        \
  hipLaunchKernelGGL((dense_pq_backward_kernel<K, NIT_, true>), dim3((unsigned)L.bsize), block, lds_q, st, gout, ent, q1, \
                     q2, gent, gq1, gq2, num, dim);                                                                    \
  hipLaunchKernelGGL((dense_shared_entity_backward_kernel<K, NIT_>), dim3((unsigned)L.num), block, lds_e, st, gout, ent,  \
                     q1, q2, gent, bsize, num, dim);
  if (ncol <= 64) {
    SMX_SHARED_LAUNCH(1)
  } else if (ncol <= 128) {
    SMX_SHARED_LAUNCH(2)
  } else {
    SMX_SHARED_LAUNCH(4)
  }
#undef SMX_SHARED_LAUNCH
  return check_launch("dist backward (shared entity rows)");
}

// ---- reverse layout, fp32: entity [B,1,.] against query [B,N,.] -------------------------------------
// (inverse queries: the tail entity is projected back through the relations and compared with one query
// row per candidate, kg_reasoning.py:252-263).  The mirror image of the per-query kernels: the entity row
// is the one that stays (LDS / registers), the query rows stream by, the query gradient is per row and the
// entity gradient is the sum over the rows.
template <int K>
__global__ __launch_bounds__(256) void dense_rev_forward_kernel(const float* __restrict__ ent, const float* __restrict__ q1,
                                                                const float* __restrict__ q2, float* __restrict__ dst,
                                                                int num, int dim, int tiles, int rows_per_tile) {
  constexpr int MUL = kind_mul(K), NQ = kind_nq(K);
  extern __shared__ float lds[];  // e1[dim] | e2[dim]
  const int b = blockIdx.x / tiles, tile = blockIdx.x - b * tiles;
  for (int d = threadIdx.x; d < dim * MUL; d += 256) lds[d] = ent[(size_t)b * dim * MUL + d];
  __syncthreads();
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int ncol = dim / 4;
  const int k1 = min(num, (tile + 1) * rows_per_tile);
  const dvec4 zero = {0.f, 0.f, 0.f, 0.f};
  for (int k = tile * rows_per_tile + wave; k < k1; k += 4) {
    const size_t r = (size_t)b * num + k;
    const dvec4* pa = reinterpret_cast<const dvec4*>(q1 + r * dim);
    const dvec4* pb = reinterpret_cast<const dvec4*>(q2 + r * dim);
    float sum = 0.f;
    for (int c = lane; c < ncol; c += kWave) {
      const dvec4 e1 = reinterpret_cast<const dvec4*>(lds)[c];
      const dvec4 e2 = MUL == 2 ? reinterpret_cast<const dvec4*>(lds + dim)[c] : zero;
      const dvec4 a = pa[c];
      const dvec4 bq = NQ == 2 ? pb[c] : zero;
#pragma unroll
      for (int x = 0; x < 4; ++x) sum += Term<K, float>::fwd(e1[x], e2[x], a[x], bq[x]);
    }
    sum = wave_sum(sum);
    if (lane == 0) dst[r] = sum;
  }
}

template <int K, int NIT>
__global__ __launch_bounds__(kPqBwdWaves * kWave) void dense_rev_backward_kernel(
    const float* __restrict__ gout, const float* __restrict__ ent, const float* __restrict__ q1,
    const float* __restrict__ q2, float* __restrict__ gent, float* __restrict__ gq1, float* __restrict__ gq2, int num,
    int dim) {
  constexpr int MUL = kind_mul(K), NQ = kind_nq(K);
  extern __shared__ float lds[];  // [waves][MUL][dim]
  const int b = blockIdx.x;
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int ncol = dim / 4;
  const size_t row_len = (size_t)dim * MUL;
  const dvec4 zero = {0.f, 0.f, 0.f, 0.f};
  dvec4 e1[NIT], e2[NIT], acc1[NIT], acc2[NIT];
  const dvec4* pe = reinterpret_cast<const dvec4*>(ent + (size_t)b * row_len);
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    const int c = min(lane + kWave * it, ncol - 1);
    e1[it] = pe[c];
    e2[it] = MUL == 2 ? pe[c + ncol] : zero;
    acc1[it] = acc2[it] = zero;
  }
  for (int k = wave; k < num; k += kPqBwdWaves) {
    const size_t r = (size_t)b * num + k;
    const float g = gout[r];
    const dvec4* pa = reinterpret_cast<const dvec4*>(q1 + r * dim);
    const dvec4* pb = reinterpret_cast<const dvec4*>(q2 + r * dim);
    dvec4 qa[NIT], qb[NIT];
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      const int c = min(lane + kWave * it, ncol - 1);
      qa[it] = pa[c];
      qb[it] = NQ == 2 ? pb[c] : zero;
    }
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      const int c = lane + kWave * it;
      if (c < ncol) {
        dvec4 g1 = zero, g2 = zero;
#pragma unroll
        for (int x = 0; x < 4; ++x) {
          float a1 = acc1[it][x], a2 = acc2[it][x], s1 = 0.f, s2 = 0.f;
          Term<K, float>::bwd(g, e1[it][x], e2[it][x], qa[it][x], qb[it][x], a1, a2, s1, s2);
          acc1[it][x] = a1;
          acc2[it][x] = a2;
          g1[x] = s1;
          g2[x] = s2;
        }
        __builtin_nontemporal_store(g1, reinterpret_cast<dvec4*>(gq1 + r * dim) + c);
        if (NQ == 2) __builtin_nontemporal_store(g2, reinterpret_cast<dvec4*>(gq2 + r * dim) + c);
      }
    }
  }
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    const int c = lane + kWave * it;
    if (c < ncol) {
      reinterpret_cast<dvec4*>(lds + (size_t)(wave * MUL + 0) * dim)[c] = acc1[it];
      if (MUL == 2) reinterpret_cast<dvec4*>(lds + (size_t)(wave * MUL + 1) * dim)[c] = acc2[it];
    }
  }
  __syncthreads();
  for (int d = threadIdx.x; d < dim * MUL; d += kPqBwdWaves * kWave) {
    const int h = d / dim, dd = d - h * dim;
    float sum = 0.f;
#pragma unroll
    for (int w = 0; w < kPqBwdWaves; ++w) sum += lds[(size_t)(w * MUL + h) * dim + dd];
    gent[(size_t)b * row_len + d] = sum;
  }
}

// entity [B,1,.] against query [B,N,.]
static bool reverse_layout(const Layout& L, const void* a, const void* b, const void* c, const void* d, const void* e,
                           const void* f, const void* g) {
  if (L.be != L.bsize || L.bc != L.bsize || L.ne != 1 || L.nc != L.num || L.num < 2) return false;
  if (L.dim % 4 != 0 || L.dim > 1024 || L.bsize * L.num > 0x7fffffffull) return false;
  return aligned16(a) && aligned16(b) && aligned16(c) && aligned16(d) && aligned16(e) && aligned16(f) && aligned16(g);
}

template <int K>
static int forward_rev(hipStream_t st, const float* ent, const float* q1, const float* q2, float* dst, const Layout& L) {
  int rows_per_tile = (int)L.num;
  while (rows_per_tile > 8 && L.bsize * ((L.num + rows_per_tile - 1) / rows_per_tile) < 8192) rows_per_tile = (rows_per_tile + 1) / 2;
  const int tiles = (int)((L.num + rows_per_tile - 1) / rows_per_tile);
  const size_t lds = (size_t)kind_mul(K) * L.dim * sizeof(float);
  hipLaunchKernelGGL((dense_rev_forward_kernel<K>), dim3((unsigned)(L.bsize * tiles)), dim3(256), lds, st, ent, q1, q2, dst,
                     (int)L.num, (int)L.dim, tiles, rows_per_tile);
  return check_launch("dist forward (reverse layout)");
}

template <int K>
static int backward_rev(hipStream_t st, const float* gout, const float* ent, const float* q1, const float* q2, float* gent,
                        float* gq1, float* gq2, const Layout& L) {
  const size_t lds = (size_t)kPqBwdWaves * kind_mul(K) * L.dim * sizeof(float);
  const dim3 grid((unsigned)L.bsize), block(kPqBwdWaves * kWave);
  const int num = (int)L.num, dim = (int)L.dim;
  const size_t ncol = L.dim / 4;
  if (ncol <= 64)
    hipLaunchKernelGGL((dense_rev_backward_kernel<K, 1>), grid, block, lds, st, gout, ent, q1, q2, gent, gq1, gq2, num, dim);
  else if (ncol <= 128)
    hipLaunchKernelGGL((dense_rev_backward_kernel<K, 2>), grid, block, lds, st, gout, ent, q1, q2, gent, gq1, gq2, num, dim);
  else
    hipLaunchKernelGGL((dense_rev_backward_kernel<K, 4>), grid, block, lds, st, gout, ent, q1, q2, gent, gq1, gq2, num, dim);
  return check_launch("dist backward (reverse layout)");
}

// entity [B,N,.] against query [B,1,.], float4-able, and small enough for the kernels above
static bool pq_layout(const Layout& L, int kind, const void* a, const void* b, const void* c, const void* d,
                      const void* e, const void* f, const void* g) {
  if (L.be != L.bsize || L.bc != L.bsize || L.ne != L.num || L.nc != 1) return false;
  if (L.dim % 4 != 0 || L.dim > 1024 || L.bsize * L.num > 0x7fffffffull || L.num > 0x7fffffffull) return false;
  (void)kind;
  return aligned16(a) && aligned16(b) && aligned16(c) && aligned16(d) && aligned16(e) && aligned16(f) && aligned16(g);
}

template <int K, bool SHARED = false>
static int forward_pq(hipStream_t st, const float* ent, const float* q1, const float* q2, float* dst, const Layout& L) {
  // enough workgroups to fill the chip, at least eight rows each when there are that many
  int rows_per_tile = (int)L.num;
  while (rows_per_tile > 8 && L.bsize * ((L.num + rows_per_tile - 1) / rows_per_tile) < 8192) rows_per_tile = (rows_per_tile + 1) / 2;
  const int tiles = (int)((L.num + rows_per_tile - 1) / rows_per_tile);
  if (L.bsize * (size_t)tiles > 0x7fffffffull) return -1;
  const size_t lds = (size_t)kind_nq(K) * L.dim * sizeof(float);
  hipLaunchKernelGGL((dense_pq_forward_kernel<K, SHARED>), dim3((unsigned)(L.bsize * tiles)), dim3(256), lds, st, ent, q1, q2, dst,
                     (int)L.num, (int)L.dim, tiles, rows_per_tile);
  return check_launch("dist forward (per-query layout)");
}

template <int K>
static int backward_pq(hipStream_t st, const float* gout, const float* ent, const float* q1, const float* q2, float* gent,
                       float* gq1, float* gq2, const Layout& L) {
  const size_t lds = (size_t)kPqBwdWaves * kind_nq(K) * L.dim * sizeof(float);
  const dim3 grid((unsigned)L.bsize), block(kPqBwdWaves * kWave);
  const int num = (int)L.num, dim = (int)L.dim;
  const size_t ncol = L.dim / 4;
  if (ncol <= 64)
    hipLaunchKernelGGL((dense_pq_backward_kernel<K, 1>), grid, block, lds, st, gout, ent, q1, q2, gent, gq1, gq2, num, dim);
  else if (ncol <= 128)
    hipLaunchKernelGGL((dense_pq_backward_kernel<K, 2>), grid, block, lds, st, gout, ent, q1, q2, gent, gq1, gq2, num, dim);
  else
    hipLaunchKernelGGL((dense_pq_backward_kernel<K, 4>), grid, block, lds, st, gout, ent, q1, q2, gent, gq1, gq2, num, dim);
  return check_launch("dist backward (per-query layout)");
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
  if constexpr (std::is_same<T, float>::value) {
    if (pq_layout(L, kind, ent, q1, q2, dst, nullptr, nullptr, nullptr)) {
      switch (kind) {
#define X(KK) \
  case KK:    \
    return forward_pq<KK>(st, ent, q1, q2, dst, L);
        SMX_FOR_EACH_KIND(X)
#undef X
      }
    }
  }
  if constexpr (std::is_same<T, float>::value) {
    if (shared_layout(L, ent, q1, q2, dst, nullptr, nullptr, nullptr)) {
      switch (kind) {
#define X(KK) \
  case KK:    \
    return forward_pq<KK, true>(st, ent, q1, q2, dst, L);
        SMX_FOR_EACH_KIND(X)
#undef X
      }
    }
    if (reverse_layout(L, ent, q1, q2, dst, nullptr, nullptr, nullptr)) {
      switch (kind) {
#define X(KK) \
  case KK:    \
    return forward_rev<KK>(st, ent, q1, q2, dst, L);
        SMX_FOR_EACH_KIND(X)
#undef X
      }
    }
  }
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
  if constexpr (std::is_same<T, float>::value) {
    if (pq_layout(L, kind, gout, ent, q1, q2, gent, gq1, gq2)) {
      switch (kind) {
#define X(KK) \
  case KK:    \
    return backward_pq<KK>(st, gout, ent, q1, q2, gent, gq1, gq2, L);
        SMX_FOR_EACH_KIND(X)
#undef X
      }
    }
  }
  if constexpr (std::is_same<T, float>::value) {
    if (shared_layout(L, gout, ent, q1, q2, gent, gq1, gq2)) {
      switch (kind) {
#define X(KK) \
  case KK:    \
    return backward_shared<KK>(st, gout, ent, q1, q2, gent, gq1, gq2, L);
        SMX_FOR_EACH_KIND(X)
#undef X
      }
    }
    if (reverse_layout(L, gout, ent, q1, q2, gent, gq1, gq2)) {
      switch (kind) {
#define X(KK) \
  case KK:    \
    return backward_rev<KK>(st, gout, ent, q1, q2, gent, gq1, gq2, L);
        SMX_FOR_EACH_KIND(X)
#undef X
      }
    }
  }
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
