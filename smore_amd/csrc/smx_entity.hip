// Entity-side backward: segmented gradient reduction with the sparse Adam row
// update fused into the same pass.  No float atomics anywhere; every sum has a
// fixed order, so two runs on the same inputs give the same bits.
//
// Replaces, per training step,
//   dist_backward_ent_kernel              smore/common/torchext/common_kernel.h:59-89
//   EmbedLookupFunc.backward / accumulate smore/common/embedding/embed_optimizer.py:63-66,146-148
//   merge_grad_list (scatter-sum)         embed_optimizer.py:45-48
//   AdamEmbedOptimizer.update_step        embed_optimizer.py:208-252
// The reference materialises a [P, row] gradient tensor, scatter-adds it into
// [U, row] and then runs ~20 row-sized tensor passes for Adam.  Here the sorted
// pair list of the segment plan is cut into fixed tiles; one wavefront walks a
// tile, recomputes each pair's entity gradient from (entity row, query row,
// upstream gradient) in registers -- or, for gradients that autograd already
// materialised, reads the pair's gradient row -- and sums it per segment.
//   * a segment that lies inside one tile is finished on the spot: the lanes
//     holding its gradient read w, m, v of that entity row, apply Adam, and
//     write the three rows back;
//   * a segment crossing a tile edge leaves one partial row per tile (tail: it
//     continues past the tile end; head: it came in from the left and ends
//     here); a second kernel adds the partials of such a segment in tile order
//     and then finishes it the same way.
// Consecutive pairs of a segment that belong to the same query (common when
// ids repeat inside one query's negatives) share one gradient evaluation: the
// derivative is linear in the upstream coefficient, so coefficients are summed
// first.
#include <cmath>

#include "smx_common.h"
#include "smx_models.h"
#include "smx_wave.h"

namespace smx {

constexpr int kSrcRows = 100;  // source = materialised gradient rows instead of a score model

__host__ __device__ constexpr int src_mul(int s) { return s == kSrcRows ? 1 : model_mul(s); }

struct AdamConsts {
  float beta1, beta2, omb1, omb2, eps, step_size, inv_sqrt_bc2;
};

struct EntityArgs {
  // plan
  const int* order;
  const int* sorted_ids;
  const int* seg_of_pos;
  const int* seg_start;
  int n_pairs;
  int tile;  // sorted positions per tile, multiple of 64
  // source: score model
  const float* q1;
  const float* q2;
  const float* score;
  const float* gscore;
  int K;
  ScoreParams p;
  // source: gradient rows
  const float* grad_rows;
  // entity table (read for the model sources, updated when adam_on)
  float* table;
  float* m;
  float* v;
  int adam_on;
  AdamConsts a;
  float* merged;  // [U, row_len] or null
  float* tail;    // [tiles, row_len]
  float* head;    // [tiles, row_len]
  int ncol;       // columns per half row (model sources) or per row (gradient rows)
};

template <int VEC> struct Pack2 {
  float v[VEC];
};

template <int VEC>
__device__ __forceinline__ Pack2<VEC> ld(const float* __restrict__ base, int col) {
  Pack2<VEC> r;
  if constexpr (VEC == 4) {
    const float4 t = reinterpret_cast<const float4*>(base)[col];
    r.v[0] = t.x;
    r.v[1] = t.y;
    r.v[2] = t.z;
    r.v[3] = t.w;
  } else {
    r.v[0] = base[col];
  }
  return r;
}

template <int VEC>
__device__ __forceinline__ void st(float* __restrict__ base, int col, const float (&x)[VEC]) {
  if constexpr (VEC == 4) {
    reinterpret_cast<float4*>(base)[col] = make_float4(x[0], x[1], x[2], x[3]);
  } else {
    base[col] = x[0];
  }
}

// Finishes one entity row: optional clamp mask, optional merged-gradient store, optional Adam.
// g1/g2 are the lane's columns of the summed gradient of the first / second half row.
template <int SRC, int VEC, int NIT>
__device__ __forceinline__ void finish_row(const EntityArgs& A, int lane, unsigned row_id, int seg,
                                           float (&g1)[NIT][VEC], float (&g2)[NIT][VEC]) {
  constexpr int MUL = src_mul(SRC);
  const int half = A.ncol * VEC;
  const size_t row_len = (size_t)half * MUL;
  float* w = A.table + (size_t)row_id * row_len;
  if (SRC != kSrcRows && A.p.reg_on) {
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      const int c = lane + 64 * it;
      if (c < A.ncol) {
        const Pack2<VEC> e1 = ld<VEC>(w, c);
#pragma unroll
        for (int x = 0; x < VEC; ++x) g1[it][x] = reg_mask(e1.v[x], g1[it][x], A.p);
        if (MUL == 2) {
          const Pack2<VEC> e2 = ld<VEC>(w + half, c);
#pragma unroll
          for (int x = 0; x < VEC; ++x) g2[it][x] = reg_mask(e2.v[x], g2[it][x], A.p);
        }
      }
    }
  }
  if (A.merged) {
    float* out = A.merged + (size_t)seg * row_len;
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      const int c = lane + 64 * it;
      if (c < A.ncol) {
        st<VEC>(out, c, g1[it]);
        if (MUL == 2) st<VEC>(out + half, c, g2[it]);
      }
    }
  }
  if (A.adam_on) {
    float* mm = A.m + (size_t)row_id * row_len;
    float* vv = A.v + (size_t)row_id * row_len;
#pragma unroll
    for (int h = 0; h < MUL; ++h) {
#pragma unroll
      for (int it = 0; it < NIT; ++it) {
        const int c = lane + 64 * it;
        if (c < A.ncol) {
          const Pack2<VEC> w0 = ld<VEC>(w + h * half, c);
          const Pack2<VEC> m0 = ld<VEC>(mm + h * half, c);
          const Pack2<VEC> v0 = ld<VEC>(vv + h * half, c);
          float wn[VEC], mn[VEC], vn[VEC];
#pragma unroll
          for (int x = 0; x < VEC; ++x) {
            const float g = h == 0 ? g1[it][x] : g2[it][x];
            mn[x] = m0.v[x] * A.a.beta1 + g * A.a.omb1;
            vn[x] = v0.v[x] * A.a.beta2 + g * g * A.a.omb2;
            const float denom = sqrtf(vn[x]) * A.a.inv_sqrt_bc2 + A.a.eps;
            wn[x] = w0.v[x] + A.a.step_size * mn[x] / denom;
          }
          st<VEC>(w + h * half, c, wn);
          st<VEC>(mm + h * half, c, mn);
          st<VEC>(vv + h * half, c, vn);
        }
      }
    }
  }
}

template <int SRC, int VEC, int NIT>
__device__ __forceinline__ void store_partial(const EntityArgs& A, float* buf, int t, int lane,
                                              const float (&g1)[NIT][VEC], const float (&g2)[NIT][VEC]) {
  constexpr int MUL = src_mul(SRC);
  const int half = A.ncol * VEC;
  float* out = buf + (size_t)t * half * MUL;
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    const int c = lane + 64 * it;
    if (c < A.ncol) {
      st<VEC>(out, c, g1[it]);
      if (MUL == 2) st<VEC>(out + half, c, g2[it]);
    }
  }
}

template <int SRC, int VEC, int NIT>
__global__ __launch_bounds__(256) void entity_tile_kernel(EntityArgs A) {
  constexpr int MUL = src_mul(SRC);
  const int lane = threadIdx.x & 63;
  const int wave = uniform(threadIdx.x >> 6);
  const int t = blockIdx.x * 4 + wave;
  const int p0 = t * A.tile;
  if (p0 >= A.n_pairs) return;  // whole wavefront leaves; no workgroup barrier is used below
  const int p1 = min(A.n_pairs, p0 + A.tile);
  const int half = A.ncol * VEC;
  const size_t row_len = (size_t)half * MUL;

  float g1[NIT][VEC], g2[NIT][VEC];
  Pack2<VEC> e1[NIT], e2[NIT];
  int cur_seg = -1;
  unsigned cur_id = 0;

  auto zero_acc = [&]() {
#pragma unroll
    for (int it = 0; it < NIT; ++it)
#pragma unroll
      for (int x = 0; x < VEC; ++x) g1[it][x] = g2[it][x] = 0.f;
  };
  auto flush = [&]() {
    const bool open_left = A.seg_start[cur_seg] < p0;
    const bool closed_right = A.seg_start[cur_seg + 1] <= p1;
    if (!closed_right)
      store_partial<SRC, VEC, NIT>(A, A.tail, t, lane, g1, g2);
    else if (open_left)
      store_partial<SRC, VEC, NIT>(A, A.head, t, lane, g1, g2);
    else
      finish_row<SRC, VEC, NIT>(A, lane, cur_id, cur_seg, g1, g2);
  };

  for (int base = p0; base < p1; base += 64) {
    const int pos = base + lane;
    const bool valid = pos < p1;
    const int my_seg = valid ? A.seg_of_pos[pos] : -1;
    const int my_id = valid ? A.sorted_ids[pos] : 0;
    const int my_pair = valid ? A.order[pos] : 0;
    float my_c0 = 0.f, my_c1 = 0.f;
    int my_b = 0;
    if (SRC != kSrcRows) {
      if (valid) {
        if constexpr (SRC != kSrcRows) ModelOps<SRC>::coef(A.gscore[my_pair], A.score[my_pair], A.p, my_c0, my_c1);
        my_b = my_pair / A.K;
      }
    }
    const int n = min(64, p1 - base);
    int j = 0;
    while (j < n) {
      const int sj = __builtin_amdgcn_readlane(my_seg, j);
      if (sj != cur_seg) {
        if (cur_seg >= 0) flush();
        cur_seg = sj;
        cur_id = (unsigned)__builtin_amdgcn_readlane(my_id, j);
        zero_acc();
        if (SRC != kSrcRows) {
          const float* pe = A.table + (size_t)cur_id * row_len;
#pragma unroll
          for (int it = 0; it < NIT; ++it) {
            const int c = lane + 64 * it;
            if (c < A.ncol) {
              e1[it] = ld<VEC>(pe, c);
              if (MUL == 2) e2[it] = ld<VEC>(pe + half, c);
            }
          }
        }
      }
      if constexpr (SRC == kSrcRows) {
        const int pj = __builtin_amdgcn_readlane(my_pair, j);
        const float* pg = A.grad_rows + (size_t)pj * row_len;
#pragma unroll
        for (int it = 0; it < NIT; ++it) {
          const int c = lane + 64 * it;
          if (c < A.ncol) {
            const Pack2<VEC> r = ld<VEC>(pg, c);
#pragma unroll
            for (int x = 0; x < VEC; ++x) g1[it][x] += r.v[x];
          }
        }
        ++j;
      } else {
        const int bj = __builtin_amdgcn_readlane(my_b, j);
        float c0 = 0.f, c1 = 0.f;
        do {  // pairs of this segment that share query bj: sum their coefficients first
          c0 += __int_as_float(__builtin_amdgcn_readlane(__float_as_int(my_c0), j));
          c1 += __int_as_float(__builtin_amdgcn_readlane(__float_as_int(my_c1), j));
          ++j;
        } while (j < n && __builtin_amdgcn_readlane(my_seg, j) == sj && __builtin_amdgcn_readlane(my_b, j) == bj);
        const float* pq1 = A.q1 + (size_t)bj * half;
        const float* pq2 = model_nq(SRC) == 2 ? A.q2 + (size_t)bj * half : pq1;
#pragma unroll
        for (int it = 0; it < NIT; ++it) {
          const int c = lane + 64 * it;
          if (c < A.ncol) {
            const Pack2<VEC> a = ld<VEC>(pq1, c);
            Pack2<VEC> b = a;
            if (model_nq(SRC) == 2) b = ld<VEC>(pq2, c);
#pragma unroll
            for (int x = 0; x < VEC; ++x) {
              const typename ModelOps<SRC>::Q q = ModelOps<SRC>::prep(a.v[x], b.v[x]);
              const float x1 = reg_apply(e1[it].v[x], A.p);
              const float x2 = MUL == 2 ? reg_apply(e2[it].v[x], A.p) : 0.f;
              ModelOps<SRC>::bwd_e(c0, c1, x1, x2, q, g1[it][x], g2[it][x]);
            }
          }
        }
      }
    }
  }
  if (cur_seg >= 0) flush();
}

// One workgroup per tile whose first segment came in from the left and ends inside the tile:
// adds that segment's partial rows (tails of the tiles it crossed, then this tile's head) in tile
// order and finishes the row.  Every other workgroup leaves at once.
template <int SRC, int VEC, int NIT, int NW>
__global__ __launch_bounds__(NW * 64) void entity_fixup_kernel(EntityArgs A) {
  constexpr int MUL = src_mul(SRC);
  extern __shared__ float lds[];
  const int t = blockIdx.x;
  const int p0 = t * A.tile;
  if (p0 == 0 || p0 >= A.n_pairs) return;
  const int p1 = min(A.n_pairs, p0 + A.tile);
  const int seg = A.seg_of_pos[p0];
  const int s0 = A.seg_start[seg], s1 = A.seg_start[seg + 1];
  if (!(s0 < p0 && s1 <= p1)) return;  // uniform over the workgroup
  const int lane = threadIdx.x & 63;
  const int wave = uniform(threadIdx.x >> 6);
  const int half = A.ncol * VEC;
  const size_t row_len = (size_t)half * MUL;
  const int ts = s0 / A.tile;
  const int n_parts = t - ts + 1;
  const int per_wave = (n_parts + NW - 1) / NW;
  const int j0 = wave * per_wave;
  const int j1 = min(n_parts, j0 + per_wave);

  float g1[NIT][VEC], g2[NIT][VEC];
#pragma unroll
  for (int it = 0; it < NIT; ++it)
#pragma unroll
    for (int x = 0; x < VEC; ++x) g1[it][x] = g2[it][x] = 0.f;
  for (int j = j0; j < j1; ++j) {
    const int tj = ts + j;
    const float* src = (tj < t ? A.tail : A.head) + (size_t)tj * row_len;
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      const int c = lane + 64 * it;
      if (c < A.ncol) {
        const Pack2<VEC> r1 = ld<VEC>(src, c);
#pragma unroll
        for (int x = 0; x < VEC; ++x) g1[it][x] += r1.v[x];
        if (MUL == 2) {
          const Pack2<VEC> r2 = ld<VEC>(src + half, c);
#pragma unroll
          for (int x = 0; x < VEC; ++x) g2[it][x] += r2.v[x];
        }
      }
    }
  }
  // combine the wavefront sums in wavefront order
  if (wave > 0) {
    float* mine = lds + (size_t)(wave - 1) * row_len;
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      const int c = lane + 64 * it;
      if (c < A.ncol) {
        st<VEC>(mine, c, g1[it]);
        if (MUL == 2) st<VEC>(mine + half, c, g2[it]);
      }
    }
  }
  __syncthreads();
  if (wave == 0) {
    for (int w = 1; w < NW; ++w) {
      const float* other = lds + (size_t)(w - 1) * row_len;
#pragma unroll
      for (int it = 0; it < NIT; ++it) {
        const int c = lane + 64 * it;
        if (c < A.ncol) {
          const Pack2<VEC> r1 = ld<VEC>(other, c);
#pragma unroll
          for (int x = 0; x < VEC; ++x) g1[it][x] += r1.v[x];
          if (MUL == 2) {
            const Pack2<VEC> r2 = ld<VEC>(other + half, c);
#pragma unroll
            for (int x = 0; x < VEC; ++x) g2[it][x] += r2.v[x];
          }
        }
      }
    }
    finish_row<SRC, VEC, NIT>(A, lane, (unsigned)A.sorted_ids[p0], seg, g1, g2);
  }
}

// ---- host side -------------------------------------------------------------------------------

static int choose_tile(size_t n_pairs) {
  // aim at >= 16k tiles so every CU holds several wavefronts; long tiles keep partial rows few
  size_t tile = ((n_pairs / 16384) + 63) / 64 * 64;
  if (tile < 64) tile = 64;
  if (tile > 256) tile = 256;
  return (int)tile;
}

static size_t entity_ws_bytes(size_t n_pairs, size_t row_len) {
  const size_t tile = (size_t)choose_tile(n_pairs);
  const size_t tiles = (n_pairs + tile - 1) / tile;
  return 2 * tiles * row_len * sizeof(float) + 256;
}

static AdamConsts adam_consts(const smx_adam_params* a) {
  AdamConsts c;
  const double bc1 = 1.0 - std::pow(a->beta1, (double)a->step);
  const double bc2 = 1.0 - std::pow(a->beta2, (double)a->step);
  c.beta1 = (float)a->beta1;
  c.beta2 = (float)a->beta2;
  c.omb1 = (float)(1.0 - a->beta1);
  c.omb2 = (float)(1.0 - a->beta2);
  c.eps = (float)a->eps;
  c.step_size = (float)(-a->lr / bc1);
  c.inv_sqrt_bc2 = (float)(1.0 / std::sqrt(bc2));
  return c;
}

template <int SRC, int VEC, int NIT>
static int launch_entity(hipStream_t st, const EntityArgs& A) {
  const int tiles = (A.n_pairs + A.tile - 1) / A.tile;
  hipLaunchKernelGGL((entity_tile_kernel<SRC, VEC, NIT>), dim3((unsigned)((tiles + 3) / 4)), dim3(256), 0, st, A);
  constexpr int NW = 8;
  const size_t lds = (size_t)(NW - 1) * A.ncol * VEC * src_mul(SRC) * sizeof(float);
  hipLaunchKernelGGL((entity_fixup_kernel<SRC, VEC, NIT, NW>), dim3((unsigned)tiles), dim3(NW * 64), lds, st, A);
  return check_launch("entity backward");
}

static int fill_plan(EntityArgs* A, const smx_plan_view* plan, void* workspace, size_t workspace_bytes, size_t row_len) {
  if (!plan || !plan->order || !plan->sorted_ids || !plan->seg_of_pos || !plan->seg_start)
    return fail(SMX_ERR_ARG, "incomplete segment plan");
  if (plan->n_pairs == 0 || plan->n_pairs > 0x7fffffffull) return fail(SMX_ERR_SHAPE, "pair count out of range");
  const size_t need = entity_ws_bytes(plan->n_pairs, row_len);
  if (!workspace || workspace_bytes < need)
    return fail(SMX_ERR_WORKSPACE, "entity workspace too small: %zu < %zu", workspace_bytes, need);
  if (reinterpret_cast<uintptr_t>(workspace) & 255u) return fail(SMX_ERR_ARG, "workspace must be 256-byte aligned");
  A->order = plan->order;
  A->sorted_ids = plan->sorted_ids;
  A->seg_of_pos = plan->seg_of_pos;
  A->seg_start = plan->seg_start;
  A->n_pairs = (int)plan->n_pairs;
  A->tile = choose_tile(plan->n_pairs);
  const size_t tiles = (plan->n_pairs + A->tile - 1) / A->tile;
  A->tail = static_cast<float*>(workspace);
  A->head = A->tail + tiles * row_len;
  return SMX_OK;
}

static int fill_adam(EntityArgs* A, float* m, float* v, const smx_adam_params* adam) {
  A->adam_on = 0;
  A->m = m;
  A->v = v;
  if (m || v || adam) {
    if (!m || !v || !adam) return fail(SMX_ERR_ARG, "Adam needs m, v and parameters together");
    if (adam->step < 1) return fail(SMX_ERR_ARG, "Adam step counter starts at 1");
    A->adam_on = 1;
    A->a = adam_consts(adam);
  }
  return SMX_OK;
}

}  // namespace smx

extern "C" {

size_t smx_entity_workspace_bytes(size_t n_pairs, size_t row_len) { return smx::entity_ws_bytes(n_pairs, row_len); }

int smx_score_backward_entity(int model, void* stream, const smx_plan_view* plan, float* table, size_t n_rows,
                              const float* q1, const float* q2, const float* score, const float* gscore, size_t B,
                              size_t K, size_t dim, const smx_score_params* params, float* merged, float* m, float* v,
                              const smx_adam_params* adam, void* workspace, size_t workspace_bytes) {
  using namespace smx;
  if (model < 0 || model >= mNumModels) return fail(SMX_ERR_KIND, "unknown score model %d", model);
  if (!table || !q1 || !score || !gscore || !params || (model_nq(model) == 2 && !q2))
    return fail(SMX_ERR_ARG, "null pointer");
  if (B == 0 || K == 0 || dim == 0 || n_rows == 0) return fail(SMX_ERR_SHAPE, "empty dimension");
  if (!merged && !m) return fail(SMX_ERR_ARG, "nothing to do: neither merged gradient nor Adam requested");
  EntityArgs A{};
  const size_t row_len = dim * model_mul(model);
  if (int rc = fill_plan(&A, plan, workspace, workspace_bytes, row_len)) return rc;
  if (plan->n_pairs != B * K) return fail(SMX_ERR_SHAPE, "plan holds %zu pairs, call has %zu", plan->n_pairs, B * K);
  if (int rc = fill_adam(&A, m, v, adam)) return rc;
  const bool vec4 = dim % 4 == 0 && aligned16(table) && aligned16(q1) && (!q2 || aligned16(q2)) &&
                    (!merged || aligned16(merged)) && (!m || (aligned16(m) && aligned16(v)));
  const int vec = vec4 ? 4 : 1;
  const size_t ncol = dim / vec;
  if (ncol > 512) return fail(SMX_ERR_SHAPE, "dim %zu not supported by the fused path", dim);
  const int need = (int)((ncol + 63) / 64);
  const int nit = need <= 1 ? 1 : (need <= 2 ? 2 : (need <= 4 ? 4 : 8));
  A.q1 = q1;
  A.q2 = q2;
  A.score = score;
  A.gscore = gscore;
  A.K = (int)K;
  A.p = ScoreParams{params->gamma, params->cen, params->reg_on, params->reg_add, params->reg_lo, params->reg_hi};
  A.table = table;
  A.merged = merged;
  A.ncol = (int)ncol;
  hipStream_t st = as_stream(stream);
#define NITS(M, V)                                   \
  switch (nit) {                                     \
    case 1: return launch_entity<M, V, 1>(st, A);    \
    case 2: return launch_entity<M, V, 2>(st, A);    \
    case 4: return launch_entity<M, V, 4>(st, A);    \
    default: return launch_entity<M, V, 8>(st, A);   \
  }
#define VECS(M)     \
  if (vec == 4) {   \
    NITS(M, 4)      \
  } else {          \
    NITS(M, 1)      \
  }
  switch (model) {
    case mL1: VECS(mL1)
    case mL2: VECS(mL2)
    case mBox: VECS(mBox)
    case mRotate: VECS(mRotate)
    case mBetaKL: VECS(mBetaKL)
  }
  return fail(SMX_ERR_KIND, "unknown score model %d", model);
}

int smx_rows_backward(void* stream, const smx_plan_view* plan, const float* grad_rows, size_t row_len, float* merged,
                      float* table, float* m, float* v, const smx_adam_params* adam, void* workspace,
                      size_t workspace_bytes) {
  using namespace smx;
  if (!grad_rows || row_len == 0) return fail(SMX_ERR_ARG, "null gradient rows");
  if (!merged && !m) return fail(SMX_ERR_ARG, "nothing to do: neither merged gradient nor Adam requested");
  EntityArgs A{};
  if (int rc = fill_plan(&A, plan, workspace, workspace_bytes, row_len)) return rc;
  if (int rc = fill_adam(&A, m, v, adam)) return rc;
  if (A.adam_on && !table) return fail(SMX_ERR_ARG, "Adam needs the weight table");
  const bool vec4 = row_len % 4 == 0 && aligned16(grad_rows) && (!merged || aligned16(merged)) &&
                    (!A.adam_on || (aligned16(table) && aligned16(m) && aligned16(v)));
  const int vec = vec4 ? 4 : 1;
  const size_t ncol = row_len / vec;
  if (ncol > 512) return fail(SMX_ERR_SHAPE, "row length %zu not supported by the fused path", row_len);
  const int need = (int)((ncol + 63) / 64);
  const int nit = need <= 1 ? 1 : (need <= 2 ? 2 : (need <= 4 ? 4 : 8));
  A.grad_rows = grad_rows;
  A.table = table;
  A.merged = merged;
  A.ncol = (int)ncol;
  A.K = 1;
  hipStream_t st = as_stream(stream);
  if (vec == 4) {
    NITS(kSrcRows, 4)
  } else {
    NITS(kSrcRows, 1)
  }
#undef VECS
#undef NITS
}

}  // extern "C"
