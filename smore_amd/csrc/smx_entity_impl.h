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
#pragma once
#include <mutex>

#include "smx_common.h"
#include "smx_models.h"
#include "smx_rowupdate.h"
#include "smx_wave.h"

namespace smx {

struct EntityArgs : RowSink {
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
  // source: gradient rows
  const float* grad_rows;
  float* tail;    // [tiles, row_len] partial rows of long segments
  float* head;    // [tiles, row_len]
  unsigned char* fix;  // [tiles] 1 where the fix-up pass has a segment to finish (written by the tile pass)
  int skip_single;  // segments of one pair were already finished by the query-backward kernel
  // sign codes written by the query-backward kernel, [n_pairs][NIT*64] bytes, or null (CODED kernels)
  const unsigned char* codes;
  // several index streams in one plan (positives + negatives of one query batch, embed_optimizer.py:155-163):
  // n_src > 1, and pair p of the plan with first[s] <= p < first[s+1] is pair (p - first[s]) of source s, which
  // has its own score / gscore / codes arrays and its own K; all sources share q1, q2.  n_src <= 1: the single
  // source described by score, gscore, codes and K above.
  int n_src;
  int first[kMaxSources + 1];
  const float* src_score[kMaxSources];
  const float* src_gscore[kMaxSources];
  const unsigned char* src_codes[kMaxSources];
  int src_K[kMaxSources];
  // Plain lookups of the same step (anchor entities, box.py:137) whose gradient autograd has materialised:
  // plan pairs from rows_first on are rows of grad_rows, [n_pairs - rows_first, row].  They sort behind the model
  // pairs of their segment and are added when the segment's row is finished.  rows_first == n_pairs: none.
  int rows_first;
  int share_rows;  // fix-up kernel: its LDS has room for one more row per wavefront, they share a segment's gradient rows
};

template <int SRC>
__device__ __forceinline__ float second_coef(float c0, const ScoreParams& p) {
  return SRC == mBox ? p.cen * c0 : 0.f;
}


// ---- runs -------------------------------------------------------------------------------------
// A "run" is a stretch of consecutive sorted positions of one segment that belong to the same
// query.  The gradient of a pair is linear in its upstream coefficient, so the coefficients of a
// run are summed first and the run costs one gradient evaluation.  Runs are handled R at a time:
// the query rows of all R runs are requested before any of them is used, which keeps R (x2) row
// loads in flight per wavefront.  For materialised gradients a "run" is one pair and the row
// requested is that pair's gradient row.

template <int R> struct RunSet {
  int key[R];    // query number (model sources) or pair number (gradient rows)
  int pair[R];   // first pair of the run (CODED: where its sign codes are)
  float c[R];    // summed coefficient (model sources)
  int n;         // valid runs
};

// Collects up to R runs from window lanes [j, j_end); my_key / my_c hold one sorted position per lane.
template <int SRC, int R, bool CODED = false>
__device__ __forceinline__ void collect_runs(RunSet<R>& rs, int& j, int j_end, int my_key, float my_c,
                                             int my_pair = 0) {
  rs.n = 0;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    rs.key[r] = 0;
    rs.pair[r] = 0;
    rs.c[r] = 0.f;
    if (j < j_end) {  // wave-uniform
      rs.n = r + 1;
      rs.key[r] = __builtin_amdgcn_readlane(my_key, j);
      if constexpr (CODED) rs.pair[r] = __builtin_amdgcn_readlane(my_pair, j);
      if constexpr (SRC == kSrcRows) {
        ++j;
      } else {
        do {
          rs.c[r] += __int_as_float(__builtin_amdgcn_readlane(__float_as_int(my_c), j));
          ++j;
        } while (j < j_end && __builtin_amdgcn_readlane(my_key, j) == rs.key[r]);
      }
    }
  }
}

template <int SRC, int VEC, int NIT, int R> struct RunRows {
  Pack2<VEC> a[R][NIT];
  Pack2<VEC> b[R][NIT];
  unsigned code[R][NIT];  // CODED: the lane's code byte per column group
};

// Requests the rows the runs need: query row(s) for the model sources, the gradient row otherwise.
template <int SRC, int VEC, int NIT, int R, bool CODED = false>
__device__ __forceinline__ void request_runs(const EntityArgs& A, int lane, const RunSet<R>& rs,
                                             RunRows<SRC, VEC, NIT, R>& rr) {
  const int half = A.ncol * VEC;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    if (r < rs.n) {
      if constexpr (CODED) {
        const unsigned char* cbase = A.codes;
        int cpair = rs.pair[r];  // wave-uniform
        if (A.n_src > 1) {
          cbase = A.src_codes[0];
#pragma unroll
          for (int s = 1; s < kMaxSources; ++s) {
            if (s < A.n_src && rs.pair[r] >= A.first[s]) {
              cbase = A.src_codes[s];
              cpair = rs.pair[r] - A.first[s];
            }
          }
        }
        const unsigned char* pc = cbase + (size_t)cpair * (NIT * 64) + lane;
#pragma unroll
        for (int it = 0; it < NIT; ++it) rr.code[r][it] = pc[64 * it];
      } else if constexpr (SRC == kSrcRows) {
        const float* pg = A.grad_rows + (size_t)rs.key[r] * half;
#pragma unroll
        for (int it = 0; it < NIT; ++it) rr.a[r][it] = ld<VEC>(pg, min(lane + 64 * it, A.ncol - 1));
      } else {
        const float* pq1 = A.q1 + (size_t)rs.key[r] * half;
#pragma unroll
        for (int it = 0; it < NIT; ++it) rr.a[r][it] = ld<VEC>(pq1, min(lane + 64 * it, A.ncol - 1));
        if constexpr (model_nq(SRC) == 2) {
          const float* pq2 = A.q2 + (size_t)rs.key[r] * half;
#pragma unroll
          for (int it = 0; it < NIT; ++it) rr.b[r][it] = ld<VEC>(pq2, min(lane + 64 * it, A.ncol - 1));
        }
      }
    }
  }
}

// Adds the gradient of the runs to the lane's accumulators.
template <int SRC, int VEC, int NIT, bool REG, int R, bool CODED = false>
__device__ __forceinline__ void apply_runs(const EntityArgs& A, const RunSet<R>& rs,
                                           const RunRows<SRC, VEC, NIT, R>& rr,
                                           const RowRegs<src_mul(SRC), VEC, NIT>& e, float (&g1)[NIT][VEC],
                                           float (&g2)[NIT][VEC]) {
  constexpr int MUL = src_mul(SRC);
#pragma unroll
  for (int r = 0; r < R; ++r) {
    if (r < rs.n) {
      float c_run = rs.c[r];
      if constexpr (!CODED && SRC == mL2)
        c_run = l2_pair_coef<VEC, NIT>(c_run, A.ncol, (int)(threadIdx.x & 63), [&](int it, int x) { return e.h[0][it].v[x]; },
                                       [&](int it, int x) { return rr.a[r][it].v[x]; });
#pragma unroll
      for (int it = 0; it < NIT; ++it) {
#pragma unroll
        for (int x = 0; x < VEC; ++x) {
          if constexpr (CODED) {
            ModelOps<SRC>::bwd_e_coded(rs.c[r], second_coef<SRC>(rs.c[r], A.p), rr.code[r][it], VEC - 1 - x, g1[it][x]);
          } else if constexpr (SRC == kSrcRows) {
            g1[it][x] += rr.a[r][it].v[x];
          } else {
            const float c0 = c_run;
            const float c1 = second_coef<SRC>(c0, A.p);
            const typename ModelOps<SRC>::Q q =
                ModelOps<SRC>::prep(rr.a[r][it].v[x], model_nq(SRC) == 2 ? rr.b[r][it].v[x] : 0.f);
            const float x1 = REG ? reg_apply(e.h[0][it].v[x], A.p) : e.h[0][it].v[x];
            const float x2 = MUL == 2 ? (REG ? reg_apply(e.h[MUL - 1][it].v[x], A.p) : e.h[MUL - 1][it].v[x]) : 0.f;
            ModelOps<SRC>::bwd_e(c0, c1, x1, x2, q, g1[it][x], g2[it][x]);
          }
        }
      }
    }
  }
}

// One sorted position per lane: the window [base, base+64) of the per-position inputs.  A position that holds
// a gradient row of a plain lookup comes back with my_pair = ~(its row number) < 0 and a zero coefficient.
template <int SRC>
__device__ __forceinline__ void load_window(const EntityArgs& A, int lane, int base, int& my_key, float& my_c,
                                            int& my_pair) {
  const int pos = min(base + lane, A.n_pairs - 1);
  if constexpr (SRC == kSrcRows) {
    my_key = my_pair = A.order[pos];
    my_c = 0.f;
  } else {
    const int plan_pair = A.order[pos];
    const bool is_row = plan_pair >= A.rows_first;
    const int pair = is_row ? 0 : plan_pair;  // a pair whose inputs exist
    my_pair = pair;
    float c1;
    if (A.n_src > 1) {  // uniform: which index stream the pair came from, and its number inside that stream
      int local = pair, K = A.src_K[0];
      const float* gs = A.src_gscore[0];
      const float* sc = A.src_score[0];
#pragma unroll
      for (int s = 1; s < kMaxSources; ++s) {
        if (s < A.n_src && pair >= A.first[s]) {
          local = pair - A.first[s];
          K = A.src_K[s];
          gs = A.src_gscore[s];
          sc = A.src_score[s];
        }
      }
      ModelOps<SRC>::coef(gs[local], sc[local], A.p, my_c, c1);
      my_key = local / K;
    } else {
      ModelOps<SRC>::coef(A.gscore[pair], A.score[pair], A.p, my_c, c1);
      my_key = pair / A.K;
    }
    if (is_row) {
      my_c = 0.f;
      my_pair = ~(plan_pair - A.rows_first);
    }
  }
}

// Lanes [j, j_end) of a window: how many of them hold gradient rows (they are the last ones of their segment).
__device__ __forceinline__ int rows_in_window(int my_pair, int j, int j_end) {
  const unsigned long long upto = j_end >= 64 ? ~0ull : ((1ull << j_end) - 1ull);
  const unsigned long long from = j >= 64 ? 0ull : ~((1ull << j) - 1ull);
  return __builtin_popcountll(__ballot(my_pair < 0) & upto & from);
}

// g += the gradient rows of the plain lookups whose numbers lanes [j0, j1) of `row_of_lane` hold, in lane order;
// kAhead rows are requested before the first is added.
template <int MUL, int VEC, int NIT, int kAhead = 4>
__device__ __forceinline__ void add_grad_rows(const EntityArgs& A, int lane, int row_of_lane, int j0, int j1,
                                              float (&g1)[NIT][VEC], float (&g2)[NIT][VEC]) {
  const int half = A.ncol * VEC;
  for (int j = j0; j < j1; j += kAhead) {  // uniform bounds
    Pack2<VEC> a[kAhead][NIT], b[kAhead][NIT];
#pragma unroll
    for (int u = 0; u < kAhead; ++u) {
      const int r = __builtin_amdgcn_readlane(row_of_lane, min(j + u, j1 - 1));
      const float* pg = A.grad_rows + (size_t)r * half * MUL;
#pragma unroll
      for (int it = 0; it < NIT; ++it) {
        const int c = min(lane + 64 * it, A.ncol - 1);
        a[u][it] = ld<VEC, true>(pg, c);
        if constexpr (MUL == 2) b[u][it] = ld<VEC, true>(pg + half, c);
      }
    }
#pragma unroll
    for (int u = 0; u < kAhead; ++u) {
      if (j + u < j1) {
#pragma unroll
        for (int it = 0; it < NIT; ++it)
#pragma unroll
          for (int x = 0; x < VEC; ++x) {
            g1[it][x] += a[u][it].v[x];
            if constexpr (MUL == 2) g2[it][x] += b[u][it].v[x];
          }
      }
    }
  }
}

// First plan position of the gradient rows at the end of segment [s0, s1) (s1 when it has none), found from the
// plan by the kernels that no longer hold the segment's window.
__device__ __forceinline__ int first_grad_row_of_segment(const EntityArgs& A, int lane, int s0, int s1) {
  int first = s1;
  for (int hi = s1; hi > s0; hi -= 64) {
    const int lo = max(s0, hi - 64);
    const int pos = lo + lane;
    const bool is_row = pos < hi && A.order[pos] >= A.rows_first;
    const unsigned long long mk = __ballot(is_row);
    if (mk == 0ull) break;
    first = lo + __builtin_ctzll(mk);
    if (__builtin_popcountll(mk) < hi - lo) break;
  }
  return first;
}

// g += the gradient rows at plan positions [first, s1), 64 at a time; of those stretches this caller takes
// number `part`, `part + parts`, ..  (a popular entity is the anchor of hundreds of queries of a batch: the
// wavefronts of a workgroup share them, and each keeps several rows in flight).  Ascending plan order per caller.
template <int MUL, int VEC, int NIT>
__device__ __forceinline__ void add_segment_grad_rows(const EntityArgs& A, int lane, int first, int s1, int part,
                                                      int parts, float (&g1)[NIT][VEC], float (&g2)[NIT][VEC]) {
  for (int base = first + part * 64; base < s1; base += parts * 64) {
    const int n_here = min(64, s1 - base);
    const int row_of_lane = A.order[base + min(lane, n_here - 1)] - A.rows_first;
    add_grad_rows<MUL, VEC, NIT, (MUL * NIT <= 2 ? 8 : 4)>(A, lane, row_of_lane, 0, n_here, g1, g2);
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
      st<VEC, true>(out, c, g1[it]);
      if (MUL == 2) st<VEC, true>(out + half, c, g2[it]);
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

// runs in flight per wavefront in the short-segment kernel / the long-segment kernel; with sign codes
// a run costs one byte per lane instead of two row loads, so more of them fit
constexpr int runs_short(bool coded) { return coded ? 4 : 2; }
constexpr int runs_long(bool coded) { return coded ? 8 : 4; }

// Short segments (at most A.short_max pairs).  The sorted pair list is cut into chunks of 64
// positions and a fixed grid of wavefronts strides over the chunks; a wavefront owns the short
// segments that START in its chunk, so its work is bounded by 64 + short_max pairs however the
// segment lengths are distributed.  The lanes fetch the chunk's per-position inputs at once; the
// wavefront then finishes one segment after the other, and while it works on one it already has
// the next one's w, m, v rows on the way (two register sets used in turn).
template <int SRC, int VEC, int NIT, bool REG, bool CODED = false>
__global__ __launch_bounds__(256) void entity_segment_kernel(EntityArgs A) {
  constexpr int MUL = src_mul(SRC);
  constexpr int R = runs_short(CODED);
  const int lane = threadIdx.x & 63;
  const int wave = uniform(threadIdx.x >> 6);
  const int n_waves = gridDim.x * 4;
  const int n_chunks = (A.n_pairs + 63) / 64;
  const int n_valid = *A.n_uniq;  // a last segment beyond this one holds the pairs whose id is outside the table: skipped
  const bool mixed = SRC != kSrcRows && A.rows_first < A.n_pairs;  // the plan also holds gradient rows of plain lookups

  for (int chunk = blockIdx.x * 4 + wave; chunk < n_chunks; chunk += n_waves) {
    const int base = chunk * 64;
    const int n_here = min(64, A.n_pairs - base);
    const int pos = base + min(lane, n_here - 1);
    const int my_seg = A.seg_of_pos[pos];
    const int my_s0 = A.seg_start[my_seg];
    const int my_s1 = A.seg_start[my_seg + 1];
    const int my_len = my_s1 - my_s0;
    bool done_elsewhere = A.skip_single && my_len == 1;  // by the pair-ordered kernel -- unless the one pair is a gradient row
    if (SRC != kSrcRows && mixed && done_elsewhere) done_elsewhere = A.order[pos] < A.rows_first;
    unsigned long long todo =
        __ballot(lane < n_here && my_s0 == pos && my_len <= A.short_max && !done_elsewhere && my_seg < n_valid);
    if (todo == 0ull) continue;
    const int my_id = A.sorted_ids[pos];

    int win_base = base;
    int my_key, my_pair;
    float my_c;
    load_window<SRC>(A, lane, win_base, my_key, my_c, my_pair);

    // finishes the segment that starts at lane i of the chunk from row state `cur`; requests the rows
    // of the segment starting at lane `nxt` (if any) into `ahead` right after this segment's first
    // run rows are requested
    auto process = [&](int i, const RowState<MUL, VEC, NIT>& cur, int nxt, RowState<MUL, VEC, NIT>& ahead) {
      const int s0 = base + i;
      const int s1 = __builtin_amdgcn_readlane(my_s1, i);
      const unsigned row_id = (unsigned)__builtin_amdgcn_readlane(my_id, i);
      const int seg = __builtin_amdgcn_readlane(my_seg, i);
      if (s1 > win_base + 64) {  // the segment runs past the window: restart the window at its first pair
        win_base = s0;
        load_window<SRC>(A, lane, win_base, my_key, my_c, my_pair);
      }
      float g1[NIT][VEC], g2[NIT][VEC];
      zero_acc<VEC, NIT>(g1, g2);
      int j = s0 - win_base;
      const int j_all = s1 - win_base;
      const int j_end = mixed ? j_all - rows_in_window(my_pair, j, j_all) : j_all;  // the model's pairs come first
      RunSet<R> rs;
      RunRows<SRC, VEC, NIT, R> rr;
      collect_runs<SRC, R, CODED>(rs, j, j_end, my_key, my_c, my_pair);
      request_runs<SRC, VEC, NIT, R, CODED>(A, lane, rs, rr);
      if (nxt >= 0) request_state<SRC, VEC, NIT>(A, lane, (unsigned)__builtin_amdgcn_readlane(my_id, nxt), ahead);
      apply_runs<SRC, VEC, NIT, REG, R, CODED>(A, rs, rr, cur.e, g1, g2);
      while (j < j_end) {
        collect_runs<SRC, R, CODED>(rs, j, j_end, my_key, my_c, my_pair);
        request_runs<SRC, VEC, NIT, R, CODED>(A, lane, rs, rr);
        apply_runs<SRC, VEC, NIT, REG, R, CODED>(A, rs, rr, cur.e, g1, g2);
      }
      auto grad_rows_of_segment = [&](float (&a1)[NIT][VEC], float (&a2)[NIT][VEC]) {
        if constexpr (SRC != kSrcRows) {
          if (j_end < j_all) add_grad_rows<MUL, VEC, NIT>(A, lane, ~my_pair, j_end, j_all, a1, a2);  // plain lookups only
        }
      };
      finish_row<SRC, VEC, NIT, REG>(A, lane, row_id, seg, g1, g2, cur.e, cur.m, cur.v, grad_rows_of_segment);
    };
    auto pop = [&]() {  // lane of the next short segment start in the chunk, -1 when none is left
      if (todo == 0ull) return -1;
      const int i = __builtin_ctzll(todo);
      todo &= todo - 1;
      return i;
    };

    RowState<MUL, VEC, NIT> sa, sb;
    int i = pop();
    request_state<SRC, VEC, NIT>(A, lane, (unsigned)__builtin_amdgcn_readlane(my_id, i), sa);
    while (true) {
      const int k = pop();
      process(i, sa, k, sb);
      if (k < 0) break;
      i = pop();
      process(k, sb, i, sa);
      if (i < 0) break;
    }
  }
}

// Long segments: the sorted pair list is cut into fixed tiles, one wavefront per tile.  The part of a
// long segment inside the tile is summed; a segment that lies wholly inside the tile is finished here,
// otherwise the sum goes to the tile's tail row (segment continues past the tile end) or head row
// (segment came in from the left and ends here).
template <int SRC, int VEC, int NIT, bool REG, bool CODED = false>
__global__ __launch_bounds__(256) void entity_tile_kernel(EntityArgs A) {
  constexpr int MUL = src_mul(SRC);
  constexpr int R = runs_long(CODED);
  const int lane = threadIdx.x & 63;
  const int wave = uniform(threadIdx.x >> 6);
  const int t = blockIdx.x * 4 + wave;
  const int p0 = t * A.tile;
  if (p0 >= A.n_pairs) return;  // whole wavefront leaves; no workgroup barrier is used below
  const int p1 = min(A.n_pairs, p0 + A.tile);
  const int n_valid = *A.n_uniq;  // the segment of ids outside the table, if there is one, is number n_valid: skipped
  const bool mixed = SRC != kSrcRows && A.rows_first < A.n_pairs;  // the plan also holds gradient rows of plain lookups
  {  // does a long segment that came in from the left end inside this tile?  The fix-up pass finishes it.
    const int sg = A.seg_of_pos[p0];
    const int b0 = A.seg_start[sg], b1 = A.seg_start[sg + 1];
    if (lane == 0) A.fix[t] = (p0 > 0 && b0 < p0 && b1 <= p1 && b1 - b0 > A.short_max && sg < n_valid) ? 1 : 0;
  }

  // most tiles hold short segments only: find that out with one parallel look and leave
  bool any_long = false;
  for (int base = p0; base < p1; base += 64) {
    const int q = min(base + lane, p1 - 1);
    const int sg = A.seg_of_pos[q];
    any_long |= __ballot(A.seg_start[sg + 1] - A.seg_start[sg] > A.short_max && sg < n_valid) != 0ull;
  }
  if (!any_long) return;

  int pos = p0;
  while (pos < p1) {
    const int seg = A.seg_of_pos[pos];
    const int s0 = A.seg_start[seg], s1 = A.seg_start[seg + 1];
    const int end = min(s1, p1);
    if (s1 - s0 > A.short_max && seg < n_valid) {
      const unsigned row_id = (unsigned)A.sorted_ids[pos];
      const bool whole = s0 >= p0 && s1 <= p1;
      RowState<MUL, VEC, NIT> st;
      if (whole) {
        request_state<SRC, VEC, NIT>(A, lane, row_id, st);
      } else if (SRC != kSrcRows && !CODED) {
        load_row<MUL, VEC, NIT>(st.e, A.table + (size_t)row_id * A.ncol * VEC * MUL, A.ncol * VEC, A.ncol, lane);
      }
      float g1[NIT][VEC], g2[NIT][VEC];
      zero_acc<VEC, NIT>(g1, g2);
      for (int base = pos; base < end; base += 64) {
        int my_key, my_pair;
        float my_c;
        load_window<SRC>(A, lane, base, my_key, my_c, my_pair);
        int j = 0;
        int j_end = min(64, end - base);
        if (mixed) j_end -= rows_in_window(my_pair, 0, j_end);  // gradient rows wait for the row's finish
        while (j < j_end) {
          RunSet<R> rs;
          RunRows<SRC, VEC, NIT, R> rr;
          collect_runs<SRC, R, CODED>(rs, j, j_end, my_key, my_c, my_pair);
          request_runs<SRC, VEC, NIT, R, CODED>(A, lane, rs, rr);
          apply_runs<SRC, VEC, NIT, REG, R, CODED>(A, rs, rr, st.e, g1, g2);
        }
      }
      if (whole) {
        auto grad_rows_of_segment = [&](float (&a1)[NIT][VEC], float (&a2)[NIT][VEC]) {
          if (mixed)
            add_segment_grad_rows<MUL, VEC, NIT>(A, lane, first_grad_row_of_segment(A, lane, s0, s1), s1, 0, 1, a1, a2);
        };
        finish_row<SRC, VEC, NIT, REG>(A, lane, row_id, seg, g1, g2, st.e, st.m, st.v, grad_rows_of_segment);
      } else if (s1 > p1)
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
  if (p0 == 0 || p0 >= A.n_pairs || A.fix[t] == 0) return;  // uniform over the workgroup; one byte decides
  const int seg = A.seg_of_pos[p0];
  const int s0 = A.seg_start[seg];
  const int lane = threadIdx.x & 63;
  const int wave = uniform(threadIdx.x >> 6);
  const int half = A.ncol * VEC;
  const size_t row_len = (size_t)half * MUL;
  const int ts = s0 / A.tile;
  const int n_parts = t - ts + 1;
  const int per_wave = (n_parts + NW - 1) / NW;
  const int j0 = wave * per_wave;
  const int j1 = min(n_parts, j0 + per_wave);

  // a few interleaved partial sums per wavefront keep several row loads in flight; they are folded
  // in a fixed order, so the result depends only on the tiling
  constexpr int ILP = NIT * MUL == 1 ? 8 : (NIT * MUL == 2 ? 4 : (NIT * MUL <= 4 ? 2 : 1));
  float acc[ILP][MUL][NIT][VEC];
#pragma unroll
  for (int k = 0; k < ILP; ++k)
#pragma unroll
    for (int h = 0; h < MUL; ++h)
#pragma unroll
      for (int it = 0; it < NIT; ++it)
#pragma unroll
        for (int x = 0; x < VEC; ++x) acc[k][h][it][x] = 0.f;
  for (int j = j0; j < j1; j += ILP) {
    RowRegs<MUL, VEC, NIT> r[ILP];
#pragma unroll
    for (int k = 0; k < ILP; ++k) {
      const int tj = ts + min(j + k, j1 - 1);
      load_row<MUL, VEC, NIT, true>(r[k], (tj < t ? A.tail : A.head) + (size_t)tj * row_len, half, A.ncol, lane);
    }
#pragma unroll
    for (int k = 0; k < ILP; ++k) {
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
      float s1 = acc[0][0][it][x], s2 = acc[0][MUL - 1][it][x];
#pragma unroll
      for (int k = 1; k < ILP; ++k) {
        s1 += acc[k][0][it][x];
        s2 += acc[k][MUL - 1][it][x];
      }
      g1[it][x] = s1;
      g2[it][x] = MUL == 2 ? s2 : 0.f;
    }
  // The segment's gradient rows of plain lookups are not part of the model's accumulators (they join after the
  // model hook and the clamp mask): with room in the LDS every wavefront sums a share of them, else the first does
  // all of them.  A.share_rows is uniform.
  const bool mixed = SRC != kSrcRows && A.rows_first < A.n_pairs;
  float h1[NIT][VEC], h2[NIT][VEC];
  zero_acc<VEC, NIT>(h1, h2);
  if (mixed && (A.share_rows || wave == 0)) {
    const int seg_end = A.seg_start[seg + 1];
    const int first = first_grad_row_of_segment(A, lane, s0, seg_end);
    add_segment_grad_rows<MUL, VEC, NIT>(A, lane, first, seg_end, A.share_rows ? wave : 0, A.share_rows ? NW : 1, h1, h2);
  }
  float* lds_rows = lds + (size_t)(NW - 1) * row_len;   // [NW - 1] rows, only there with A.share_rows
  // combine the wavefront sums in wavefront order
  if (wave > 0) {
    store_partial<SRC, VEC, NIT>(A, lds, wave - 1, lane, g1, g2);
    if (mixed && A.share_rows) store_partial<SRC, VEC, NIT>(A, lds_rows, wave - 1, lane, h1, h2);
  }
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
    if (mixed && A.share_rows) {
      for (int w = 1; w < NW; ++w) {
        RowRegs<MUL, VEC, NIT> o;
        load_row<MUL, VEC, NIT>(o, lds_rows + (size_t)(w - 1) * row_len, half, A.ncol, lane);
#pragma unroll
        for (int it = 0; it < NIT; ++it)
#pragma unroll
          for (int x = 0; x < VEC; ++x) {
            h1[it][x] += o.h[0][it].v[x];
            if (MUL == 2) h2[it][x] += o.h[MUL - 1][it].v[x];
          }
      }
    }
    const unsigned row_id = (unsigned)A.sorted_ids[p0];
    RowRegs<MUL, VEC, NIT> e, m0, v0;
    if (REG || A.adam_on || SRC == mBetaKL)
      load_row<MUL, VEC, NIT, true>(e, A.table + (size_t)row_id * row_len, half, A.ncol, lane);
    if (A.adam_on == kOptAdam) load_row<MUL, VEC, NIT, true>(m0, A.m + (size_t)row_id * row_len, half, A.ncol, lane);
    if (A.adam_on && A.adam_on != kOptSgd && !A.squeeze)
      load_row<MUL, VEC, NIT, true>(v0, A.v + (size_t)row_id * row_len, half, A.ncol, lane);
    auto grad_rows_of_segment = [&](float (&a1)[NIT][VEC], float (&a2)[NIT][VEC]) {
      if (mixed) {
#pragma unroll
        for (int it = 0; it < NIT; ++it)
#pragma unroll
          for (int x = 0; x < VEC; ++x) {
            a1[it][x] += h1[it][x];
            if (MUL == 2) a2[it][x] += h2[it][x];
          }
      }
    };
    finish_row<SRC, VEC, NIT, REG>(A, lane, row_id, seg, g1, g2, e, m0, v0, grad_rows_of_segment);
  }
}

// Workgroups of 256 threads of `kernel` the current device keeps resident (asked once per kernel and device).
template <class K>
unsigned resident_blocks(K kernel) {
  static std::mutex mu;                 // one table per instantiation, i.e. per kernel
  static unsigned cached[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256u * 8u;
  std::lock_guard<std::mutex> lock(mu);
  if (cached[dev] == 0) {
    int cus = 0, per_cu = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, 256, 0) != hipSuccess || cus <= 0 || per_cu <= 0)
      return 256u * 8u;
    cached[dev] = (unsigned)cus * (unsigned)per_cu;
  }
  return cached[dev];
}

template <int SRC, int VEC, int NIT, bool REG>
int launch_entity_reg(hipStream_t st, const EntityArgs& A) {
  const unsigned tiles = (unsigned)((A.n_pairs + A.tile - 1) / A.tile);
  // short segments: a fixed grid of wavefronts strides over the segment list (its length lives on the device)
  // (as many workgroups as the chip holds at once: a second wave of workgroups would run half empty)
  const unsigned want_blocks = (unsigned)((A.n_pairs + 255) / 256);
  bool coded = false;
  if constexpr (SRC != kSrcRows && model_coded(SRC) && !REG) coded = A.codes != nullptr;
  if (coded) {
    if constexpr (SRC != kSrcRows && model_coded(SRC) && !REG) {
      const unsigned seg_blocks = min(want_blocks, resident_blocks(entity_segment_kernel<SRC, VEC, NIT, REG, true>));
      hipLaunchKernelGGL((entity_segment_kernel<SRC, VEC, NIT, REG, true>), dim3(seg_blocks), dim3(256), 0, st, A);
      hipLaunchKernelGGL((entity_tile_kernel<SRC, VEC, NIT, REG, true>), dim3((tiles + 3) / 4), dim3(256), 0, st, A);
    }
  } else {
    const unsigned seg_blocks = min(want_blocks, resident_blocks(entity_segment_kernel<SRC, VEC, NIT, REG>));
    hipLaunchKernelGGL((entity_segment_kernel<SRC, VEC, NIT, REG>), dim3(seg_blocks), dim3(256), 0, st, A);
    hipLaunchKernelGGL((entity_tile_kernel<SRC, VEC, NIT, REG>), dim3((tiles + 3) / 4), dim3(256), 0, st, A);
  }
  const size_t row_bytes = (size_t)A.ncol * VEC * src_mul(SRC) * sizeof(float);
  const bool mixed = SRC != kSrcRows && A.rows_first < A.n_pairs;
  EntityArgs F = A;
  if (7 * row_bytes <= 60 * 1024) {
    F.share_rows = mixed && 14 * row_bytes <= 60 * 1024;
    hipLaunchKernelGGL((entity_fixup_kernel<SRC, VEC, NIT, 8, REG>), dim3(tiles), dim3(8 * 64),
                       (F.share_rows ? 14 : 7) * row_bytes, st, F);
  } else {
    F.share_rows = mixed && 6 * row_bytes <= 60 * 1024;
    hipLaunchKernelGGL((entity_fixup_kernel<SRC, VEC, NIT, 4, REG>), dim3(tiles), dim3(4 * 64),
                       (F.share_rows ? 6 : 3) * row_bytes, st, F);
  }
  return check_launch("entity backward");
}

template <int SRC, int VEC, int NIT>
int launch_entity(hipStream_t st, const EntityArgs& A) {
  if constexpr (SRC == mBetaKL) {
    if (A.p.reg_on) return launch_entity_reg<SRC, VEC, NIT, true>(st, A);
  }
  return launch_entity_reg<SRC, VEC, NIT, false>(st, A);
}

// Instantiated once per source in its own translation unit (smx_entity_inst_*.hip).
template <int SRC>
int entity_dispatch(hipStream_t st, const EntityArgs& A, int vec, int nit) {
  if (vec == 4) {
    switch (nit) {
      case 1: return launch_entity<SRC, 4, 1>(st, A);
      case 2: return launch_entity<SRC, 4, 2>(st, A);
      case 4: return launch_entity<SRC, 4, 4>(st, A);
      default: return launch_entity<SRC, 4, 8>(st, A);
    }
  }
  switch (nit) {
    case 1: return launch_entity<SRC, 1, 1>(st, A);
    case 2: return launch_entity<SRC, 1, 2>(st, A);
    default: return launch_entity<SRC, 1, 4>(st, A);
  }
}

}  // namespace smx
