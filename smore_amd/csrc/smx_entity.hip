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
  const long long* uniq;
  const int* n_uniq;
  int n_pairs;
  int tile;        // sorted positions per tile of the long-segment pass, multiple of 64
  int short_max;   // segments of at most this many pairs are finished by one wavefront
  // source: score model
  const float* q1;
  const float* q2;
  const float* score;
  const float* gscore;
  int K;
  ScoreParams p;
  float* meta_c;  // [P] upstream coefficient of every sorted position
  int* meta_b;    // [P] query number of every sorted position
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

// The lane's columns of one table row (both halves for the two-half models).
template <int MUL, int VEC, int NIT> struct RowRegs {
  Pack2<VEC> h[MUL][NIT];
};

template <int MUL, int VEC, int NIT>
__device__ __forceinline__ void load_row(RowRegs<MUL, VEC, NIT>& r, const float* __restrict__ base, int half, int ncol,
                                         int lane) {
#pragma unroll
  for (int h = 0; h < MUL; ++h)
#pragma unroll
    for (int it = 0; it < NIT; ++it) r.h[h][it] = ld<VEC>(base + h * half, min(lane + 64 * it, ncol - 1));
}

// Coefficient on the second accumulator (BOX: inside distance) from the first.
template <int SRC>
__device__ __forceinline__ float second_coef(float c0, const ScoreParams& p) {
  return SRC == mBox ? p.cen * c0 : 0.f;
}

// Adds the gradient of one run -- pairs of one segment that share query b, coefficients already
// summed into c0 -- to the lane's accumulators.
template <int SRC, int VEC, int NIT, bool REG>
__device__ __forceinline__ void add_run(const EntityArgs& A, int lane, int b, float c0,
                                        const RowRegs<src_mul(SRC), VEC, NIT>& e, float (&g1)[NIT][VEC],
                                        float (&g2)[NIT][VEC]) {
  if constexpr (SRC != kSrcRows) {
    constexpr int MUL = src_mul(SRC);
    const int half = A.ncol * VEC;
    const float c1 = second_coef<SRC>(c0, A.p);
    const float* pq1 = A.q1 + (size_t)b * half;
    const float* pq2 = model_nq(SRC) == 2 ? A.q2 + (size_t)b * half : pq1;
    Pack2<VEC> qa[NIT], qb[NIT];
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      const int c = min(lane + 64 * it, A.ncol - 1);
      qa[it] = ld<VEC>(pq1, c);
      if (model_nq(SRC) == 2) qb[it] = ld<VEC>(pq2, c);
    }
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
#pragma unroll
      for (int x = 0; x < VEC; ++x) {
        const typename ModelOps<SRC>::Q q = ModelOps<SRC>::prep(qa[it].v[x], model_nq(SRC) == 2 ? qb[it].v[x] : 0.f);
        const float x1 = REG ? reg_apply(e.h[0][it].v[x], A.p) : e.h[0][it].v[x];
        const float x2 = MUL == 2 ? (REG ? reg_apply(e.h[MUL - 1][it].v[x], A.p) : e.h[MUL - 1][it].v[x]) : 0.f;
        ModelOps<SRC>::bwd_e(c0, c1, x1, x2, q, g1[it][x], g2[it][x]);
      }
    }
  }
}

// Adds one materialised gradient row.
template <int VEC, int NIT>
__device__ __forceinline__ void add_grad_row(const EntityArgs& A, int lane, int pair, float (&g1)[NIT][VEC]) {
  const float* pg = A.grad_rows + (size_t)pair * A.ncol * VEC;
  Pack2<VEC> r[NIT];
#pragma unroll
  for (int it = 0; it < NIT; ++it) r[it] = ld<VEC>(pg, min(lane + 64 * it, A.ncol - 1));
#pragma unroll
  for (int it = 0; it < NIT; ++it)
#pragma unroll
    for (int x = 0; x < VEC; ++x) g1[it][x] += r[it].v[x];
}

// Finishes one entity row: clamp mask, merged-gradient store, Adam.  g1/g2 are the lane's columns of
// the summed gradient of the first / second half row; w, m0, v0 the row's current weights and moments
// (w is always valid for the model sources -- it is the entity row the gradient was computed from).
template <int SRC, int VEC, int NIT, bool REG>
__device__ __forceinline__ void finish_row(const EntityArgs& A, int lane, unsigned row_id, int seg,
                                           float (&g1)[NIT][VEC], float (&g2)[NIT][VEC],
                                           const RowRegs<src_mul(SRC), VEC, NIT>& w,
                                           const RowRegs<src_mul(SRC), VEC, NIT>& m0,
                                           const RowRegs<src_mul(SRC), VEC, NIT>& v0) {
  constexpr int MUL = src_mul(SRC);
  const int half = A.ncol * VEC;
  const size_t row_len = (size_t)half * MUL;
  if (REG) {
#pragma unroll
    for (int it = 0; it < NIT; ++it)
#pragma unroll
      for (int x = 0; x < VEC; ++x) {
        g1[it][x] = reg_mask(w.h[0][it].v[x], g1[it][x], A.p);
        if (MUL == 2) g2[it][x] = reg_mask(w.h[MUL - 1][it].v[x], g2[it][x], A.p);
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
    float* pw = A.table + (size_t)row_id * row_len;
    float* pm = A.m + (size_t)row_id * row_len;
    float* pv = A.v + (size_t)row_id * row_len;
#pragma unroll
    for (int h = 0; h < MUL; ++h) {
#pragma unroll
      for (int it = 0; it < NIT; ++it) {
        const int c = lane + 64 * it;
        if (c < A.ncol) {
          float wn[VEC], mn[VEC], vn[VEC];
#pragma unroll
          for (int x = 0; x < VEC; ++x) {
            const float g = h == 0 ? g1[it][x] : g2[it][x];
            mn[x] = m0.h[h][it].v[x] * A.a.beta1 + g * A.a.omb1;
            vn[x] = v0.h[h][it].v[x] * A.a.beta2 + g * g * A.a.omb2;
            const float denom = sqrtf(vn[x]) * A.a.inv_sqrt_bc2 + A.a.eps;
            wn[x] = w.h[h][it].v[x] + A.a.step_size * mn[x] / denom;
          }
          st<VEC>(pw + h * half, c, wn);
          st<VEC>(pm + h * half, c, mn);
          st<VEC>(pv + h * half, c, vn);
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

template <int VEC, int NIT>
__device__ __forceinline__ void zero_acc(float (&g1)[NIT][VEC], float (&g2)[NIT][VEC]) {
#pragma unroll
  for (int it = 0; it < NIT; ++it)
#pragma unroll
    for (int x = 0; x < VEC; ++x) g1[it][x] = g2[it][x] = 0.f;
}

// Sorted copy of what the entity pass needs per pair, so that the pass reads it contiguously:
// meta_c[pos] = d loss / d distance of the pair at sorted position pos, meta_b[pos] = its query.
template <int SRC>
__global__ __launch_bounds__(256) void entity_meta_kernel(EntityArgs A) {
  const int pos = blockIdx.x * blockDim.x + threadIdx.x;
  if (pos >= A.n_pairs) return;
  if constexpr (SRC != kSrcRows) {
    const int pair = A.order[pos];
    float c0, c1;
    ModelOps<SRC>::coef(A.gscore[pair], A.score[pair], A.p, c0, c1);
    A.meta_c[pos] = c0;
    A.meta_b[pos] = pair / A.K;
  }
}

// Walks `len` sorted positions starting at `first` that all belong to one segment and adds their
// gradient to g1/g2: run by run for the model sources, row by row for materialised gradients.
template <int SRC, int VEC, int NIT, bool REG>
__device__ __forceinline__ void add_positions(const EntityArgs& A, int lane, int first, int len,
                                              const RowRegs<src_mul(SRC), VEC, NIT>& e, float (&g1)[NIT][VEC],
                                              float (&g2)[NIT][VEC]) {
  for (int base = 0; base < len; base += 64) {
    const int n = min(64, len - base);
    const int pos = first + base + min(lane, n - 1);
    if constexpr (SRC == kSrcRows) {
      const int my_pair = A.order[pos];
      for (int j = 0; j < n; ++j) add_grad_row<VEC, NIT>(A, lane, __builtin_amdgcn_readlane(my_pair, j), g1);
    } else {
      const float my_c = A.meta_c[pos];
      const int my_b = A.meta_b[pos];
      int j = 0;
      while (j < n) {
        const int bj = __builtin_amdgcn_readlane(my_b, j);
        float c0 = 0.f;
        do {  // pairs that share query bj: the gradient is linear in the coefficient, sum it first
          c0 += __int_as_float(__builtin_amdgcn_readlane(__float_as_int(my_c), j));
          ++j;
        } while (j < n && __builtin_amdgcn_readlane(my_b, j) == bj);
        add_run<SRC, VEC, NIT, REG>(A, lane, bj, c0, e, g1, g2);
      }
    }
  }
}

// Short segments (at most A.short_max pairs): one wavefront per segment, grid-stride over segments.
template <int SRC, int VEC, int NIT, bool REG>
__global__ __launch_bounds__(256) void entity_segment_kernel(EntityArgs A) {
  constexpr int MUL = src_mul(SRC);
  const int lane = threadIdx.x & 63;
  const int wave = uniform(threadIdx.x >> 6);
  const int n_waves = gridDim.x * 4;
  const int n_uniq = *A.n_uniq;
  const int half = A.ncol * VEC;
  const size_t row_len = (size_t)half * MUL;
  for (int u = blockIdx.x * 4 + wave; u < n_uniq; u += n_waves) {
    const int s0 = A.seg_start[u], s1 = A.seg_start[u + 1];
    if (s1 - s0 > A.short_max) continue;
    const unsigned row_id = (unsigned)A.uniq[u];
    RowRegs<MUL, VEC, NIT> e, m0, v0;
    if (SRC != kSrcRows || A.adam_on) load_row<MUL, VEC, NIT>(e, A.table + (size_t)row_id * row_len, half, A.ncol, lane);
    if (A.adam_on) {
      load_row<MUL, VEC, NIT>(m0, A.m + (size_t)row_id * row_len, half, A.ncol, lane);
      load_row<MUL, VEC, NIT>(v0, A.v + (size_t)row_id * row_len, half, A.ncol, lane);
    }
    float g1[NIT][VEC], g2[NIT][VEC];
    zero_acc<VEC, NIT>(g1, g2);
    add_positions<SRC, VEC, NIT, REG>(A, lane, s0, s1 - s0, e, g1, g2);
    finish_row<SRC, VEC, NIT, REG>(A, lane, row_id, u, g1, g2, e, m0, v0);
  }
}

// Long segments: the sorted pair list is cut into fixed tiles, one wavefront per tile.  The part of a
// long segment inside the tile is summed; a segment that lies wholly inside the tile is finished here,
// otherwise the sum goes to the tile's tail row (segment continues past the tile end) or head row
// (segment came in from the left and ends here).
template <int SRC, int VEC, int NIT, bool REG>
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

  // most tiles hold short segments only: find that out with one parallel look and leave
  bool any_long = false;
  for (int base = p0; base < p1; base += 64) {
    const int q = min(base + lane, p1 - 1);
    const int sg = A.seg_of_pos[q];
    any_long |= __ballot(A.seg_start[sg + 1] - A.seg_start[sg] > A.short_max) != 0ull;
  }
  if (!any_long) return;

  int pos = p0;
  while (pos < p1) {
    const int seg = A.seg_of_pos[pos];
    const int s0 = A.seg_start[seg], s1 = A.seg_start[seg + 1];
    const int end = min(s1, p1);
    if (s1 - s0 > A.short_max) {
      const unsigned row_id = (unsigned)A.sorted_ids[pos];
      const bool whole = s0 >= p0 && s1 <= p1;
      RowRegs<MUL, VEC, NIT> e, m0, v0;
      if (SRC != kSrcRows || (whole && A.adam_on))
        load_row<MUL, VEC, NIT>(e, A.table + (size_t)row_id * row_len, half, A.ncol, lane);
      if (whole && A.adam_on) {
        load_row<MUL, VEC, NIT>(m0, A.m + (size_t)row_id * row_len, half, A.ncol, lane);
        load_row<MUL, VEC, NIT>(v0, A.v + (size_t)row_id * row_len, half, A.ncol, lane);
      }
      float g1[NIT][VEC], g2[NIT][VEC];
      zero_acc<VEC, NIT>(g1, g2);
      add_positions<SRC, VEC, NIT, REG>(A, lane, pos, end - pos, e, g1, g2);
      if (whole)
        finish_row<SRC, VEC, NIT, REG>(A, lane, row_id, seg, g1, g2, e, m0, v0);
      else if (s1 > p1)
        store_partial<SRC, VEC, NIT>(A, A.tail, t, lane, g1, g2);
      else
        store_partial<SRC, VEC, NIT>(A, A.head, t, lane, g1, g2);
    }
    pos = end;
  }
}

// One workgroup per tile whose first segment is long, came in from the left and ends inside the tile:
// adds that segment's partial rows (tails of the tiles it crossed, then this tile's head) in tile
// order and finishes the row.  Every other workgroup leaves at once.
template <int SRC, int VEC, int NIT, int NW, bool REG>
__global__ __launch_bounds__(NW * 64) void entity_fixup_kernel(EntityArgs A) {
  constexpr int MUL = src_mul(SRC);
  extern __shared__ float lds[];
  const int t = blockIdx.x;
  const int p0 = t * A.tile;
  if (p0 == 0 || p0 >= A.n_pairs) return;
  const int p1 = min(A.n_pairs, p0 + A.tile);
  const int seg = A.seg_of_pos[p0];
  const int s0 = A.seg_start[seg], s1 = A.seg_start[seg + 1];
  if (!(s0 < p0 && s1 <= p1 && s1 - s0 > A.short_max)) return;  // uniform over the workgroup
  const int lane = threadIdx.x & 63;
  const int wave = uniform(threadIdx.x >> 6);
  const int half = A.ncol * VEC;
  const size_t row_len = (size_t)half * MUL;
  const int ts = s0 / A.tile;
  const int n_parts = t - ts + 1;
  const int per_wave = (n_parts + NW - 1) / NW;
  const int j0 = wave * per_wave;
  const int j1 = min(n_parts, j0 + per_wave);

  // four interleaved partial sums per wavefront keep four row loads in flight; they are folded in a
  // fixed order, so the result depends only on the tiling
  float acc[4][MUL][NIT][VEC];
#pragma unroll
  for (int k = 0; k < 4; ++k)
#pragma unroll
    for (int h = 0; h < MUL; ++h)
#pragma unroll
      for (int it = 0; it < NIT; ++it)
#pragma unroll
        for (int x = 0; x < VEC; ++x) acc[k][h][it][x] = 0.f;
  for (int j = j0; j < j1; j += 4) {
    RowRegs<MUL, VEC, NIT> r[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int tj = ts + min(j + k, j1 - 1);
      load_row<MUL, VEC, NIT>(r[k], (tj < t ? A.tail : A.head) + (size_t)tj * row_len, half, A.ncol, lane);
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      if (j + k < j1) {
#pragma unroll
        for (int h = 0; h < MUL; ++h)
#pragma unroll
          for (int it = 0; it < NIT; ++it)
#pragma unroll
            for (int x = 0; x < VEC; ++x) acc[k][h][it][x] += r[k].h[h][it].v[x];
      }
    }
  }
  float g1[NIT][VEC], g2[NIT][VEC];
#pragma unroll
  for (int it = 0; it < NIT; ++it)
#pragma unroll
    for (int x = 0; x < VEC; ++x) {
      g1[it][x] = (acc[0][0][it][x] + acc[1][0][it][x]) + (acc[2][0][it][x] + acc[3][0][it][x]);
      g2[it][x] = MUL == 2 ? (acc[0][MUL - 1][it][x] + acc[1][MUL - 1][it][x]) +
                                 (acc[2][MUL - 1][it][x] + acc[3][MUL - 1][it][x])
                           : 0.f;
    }
  // combine the wavefront sums in wavefront order
  if (wave > 0) store_partial<SRC, VEC, NIT>(A, lds, wave - 1, lane, g1, g2);
  __syncthreads();
  if (wave == 0) {
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
    const unsigned row_id = (unsigned)A.sorted_ids[p0];
    RowRegs<MUL, VEC, NIT> e, m0, v0;
    if (REG || A.adam_on) load_row<MUL, VEC, NIT>(e, A.table + (size_t)row_id * row_len, half, A.ncol, lane);
    if (A.adam_on) {
      load_row<MUL, VEC, NIT>(m0, A.m + (size_t)row_id * row_len, half, A.ncol, lane);
      load_row<MUL, VEC, NIT>(v0, A.v + (size_t)row_id * row_len, half, A.ncol, lane);
    }
    finish_row<SRC, VEC, NIT, REG>(A, lane, row_id, seg, g1, g2, e, m0, v0);
  }
}

// ---- host side -------------------------------------------------------------------------------

constexpr int kTile = 256;      // sorted positions per tile of the long-segment pass
constexpr int kShortMax = 64;   // longest segment one wavefront finishes on its own

static size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

struct EntityScratch {
  size_t tail_off, head_off, meta_c_off, meta_b_off, total;
};

static EntityScratch entity_scratch(size_t n_pairs, size_t row_len) {
  const size_t tiles = (n_pairs + kTile - 1) / kTile;
  EntityScratch s;
  s.tail_off = 0;
  s.head_off = align256(tiles * row_len * sizeof(float));
  s.meta_c_off = s.head_off + align256(tiles * row_len * sizeof(float));
  s.meta_b_off = s.meta_c_off + align256(n_pairs * sizeof(float));
  s.total = s.meta_b_off + align256(n_pairs * sizeof(int));
  return s;
}

static size_t entity_ws_bytes(size_t n_pairs, size_t row_len) { return entity_scratch(n_pairs, row_len).total; }

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

template <int SRC, int VEC, int NIT, bool REG>
static int launch_entity_reg(hipStream_t st, const EntityArgs& A) {
  const unsigned tiles = (unsigned)((A.n_pairs + A.tile - 1) / A.tile);
  if (SRC != kSrcRows)
    hipLaunchKernelGGL((entity_meta_kernel<SRC>), dim3((unsigned)((A.n_pairs + 255) / 256)), dim3(256), 0, st, A);
  // short segments: a fixed grid of wavefronts strides over the segment list (its length lives on the device)
  unsigned seg_blocks = (unsigned)((A.n_pairs + 3) / 4);
  if (seg_blocks > 256u * 8u) seg_blocks = 256u * 8u;
  hipLaunchKernelGGL((entity_segment_kernel<SRC, VEC, NIT, REG>), dim3(seg_blocks), dim3(256), 0, st, A);
  hipLaunchKernelGGL((entity_tile_kernel<SRC, VEC, NIT, REG>), dim3((tiles + 3) / 4), dim3(256), 0, st, A);
  const size_t row_bytes = (size_t)A.ncol * VEC * src_mul(SRC) * sizeof(float);
  if (15 * row_bytes <= 60 * 1024)
    hipLaunchKernelGGL((entity_fixup_kernel<SRC, VEC, NIT, 16, REG>), dim3(tiles), dim3(16 * 64), 15 * row_bytes, st, A);
  else
    hipLaunchKernelGGL((entity_fixup_kernel<SRC, VEC, NIT, 4, REG>), dim3(tiles), dim3(4 * 64), 3 * row_bytes, st, A);
  return check_launch("entity backward");
}

template <int SRC, int VEC, int NIT>
static int launch_entity(hipStream_t st, const EntityArgs& A) {
  if constexpr (SRC == mBetaKL) {
    if (A.p.reg_on) return launch_entity_reg<SRC, VEC, NIT, true>(st, A);
  }
  return launch_entity_reg<SRC, VEC, NIT, false>(st, A);
}

static int fill_plan(EntityArgs* A, const smx_plan_view* plan, void* workspace, size_t workspace_bytes, size_t row_len) {
  if (!plan || !plan->order || !plan->sorted_ids || !plan->seg_of_pos || !plan->seg_start || !plan->uniq ||
      !plan->n_uniq)
    return fail(SMX_ERR_ARG, "incomplete segment plan");
  if (plan->n_pairs == 0 || plan->n_pairs > 0x7fffffffull) return fail(SMX_ERR_SHAPE, "pair count out of range");
  const EntityScratch sc = entity_scratch(plan->n_pairs, row_len);
  if (!workspace || workspace_bytes < sc.total)
    return fail(SMX_ERR_WORKSPACE, "entity workspace too small: %zu < %zu", workspace_bytes, sc.total);
  if (reinterpret_cast<uintptr_t>(workspace) & 255u) return fail(SMX_ERR_ARG, "workspace must be 256-byte aligned");
  A->order = plan->order;
  A->sorted_ids = plan->sorted_ids;
  A->seg_of_pos = plan->seg_of_pos;
  A->seg_start = plan->seg_start;
  A->uniq = reinterpret_cast<const long long*>(plan->uniq);
  A->n_uniq = plan->n_uniq;
  A->n_pairs = (int)plan->n_pairs;
  A->tile = kTile;
  A->short_max = kShortMax;
  char* ws = static_cast<char*>(workspace);
  A->tail = reinterpret_cast<float*>(ws + sc.tail_off);
  A->head = reinterpret_cast<float*>(ws + sc.head_off);
  A->meta_c = reinterpret_cast<float*>(ws + sc.meta_c_off);
  A->meta_b = reinterpret_cast<int*>(ws + sc.meta_b_off);
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
  if (params->reg_on && model != mBetaKL)
    return fail(SMX_ERR_ARG, "the entity clamp prologue exists for the beta_kl model only");
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
