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
#include <map>
#include <mutex>
#include <utility>

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
  int chunk;       // sorted positions a wavefront of the short-segment pass owns per turn: 64, or a smaller power of
                   // two for a short list (a step whose negatives are shared sorts a couple of thousand ids: with 64
                   // positions per wavefront two dozen wavefronts would finish their segments one after the other)
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
  int* fix_list;   // [tiles] numbers of the tiles the fix-up pass has a segment to finish for (appended by the tile pass)
  int* fix_count;  // how many; cleared by the segment pass, which runs first
  int skip_single;  // segments of one pair were already finished by the query-backward kernel
  // sign codes written by the query-backward kernel, [n_pairs][NIT*64] bytes, or null (CODED kernels)
  const unsigned char* codes;
  // several index streams in one plan (positives + negatives of one query batch, embed_optimizer.py:155-163):
  // n_src > 1, and pair p of the plan with first[s] <= p < first[s+1] is pair (p - first[s]) of source s, which
  // has its own score / gscore / codes arrays and its own K; its queries are rows src_q0[s] .. of q1, q2 (all
  // sources the same rows when they belong to one query batch).  n_src <= 1: the single source described by
  // score, gscore, codes and K above.
  int n_src;
  int first[kMaxSources + 1];
  int src_q0[kMaxSources];
  const float* src_score[kMaxSources];
  const float* src_gscore[kMaxSources];
  const unsigned char* src_codes[kMaxSources];
  int src_K[kMaxSources];
  // Union queries: q1 / q2 hold U branch rows per query; a pair's gradient is taken against the branch that gave
  // its logit (the first maximal one, as torch.max routes it): winner[pair], per source.  U == 1: no such array.
  int U;
  const unsigned char* winner;
  const unsigned char* src_winner[kMaxSources];
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
  float c[R];    // summed coefficient (model sources)
  int n;         // valid runs
};

// Collects up to R runs from window lanes [j, j_end); my_key / my_c hold one sorted position per lane.
template <int SRC, int R>
__device__ __forceinline__ void collect_runs(RunSet<R>& rs, int& j, int j_end, int my_key, float my_c) {
  rs.n = 0;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    rs.key[r] = 0;
    rs.c[r] = 0.f;
    if (j < j_end) {  // wave-uniform
      rs.n = r + 1;
      rs.key[r] = __builtin_amdgcn_readlane(my_key, j);
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
};

// Requests the rows the runs need: query row(s) for the model sources, the gradient row otherwise.
template <int SRC, int VEC, int NIT, int R>
__device__ __forceinline__ void request_runs(const EntityArgs& A, int lane, const RunSet<R>& rs,
                                             RunRows<SRC, VEC, NIT, R>& rr) {
  const int half = A.ncol * VEC;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    if (r < rs.n) {
      if constexpr (SRC == kSrcRows) {
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
template <int SRC, int VEC, int NIT, bool REG, int R>
__device__ __forceinline__ void apply_runs(const EntityArgs& A, const RunSet<R>& rs,
                                           const RunRows<SRC, VEC, NIT, R>& rr,
                                           const RowRegs<src_mul(SRC), VEC, NIT>& e, float (&g1)[NIT][VEC],
                                           float (&g2)[NIT][VEC]) {
  constexpr int MUL = src_mul(SRC);
#pragma unroll
  for (int r = 0; r < R; ++r) {
    if (r < rs.n) {
      float c_run = rs.c[r];
      if constexpr (SRC == mL2)
        c_run = l2_pair_coef<VEC, NIT>(c_run, A.ncol, (int)(threadIdx.x & 63), [&](int it, int x) { return e.h[0][it].v[x]; },
                                       [&](int it, int x) { return rr.a[r][it].v[x]; });
#pragma unroll
      for (int it = 0; it < NIT; ++it) {
#pragma unroll
        for (int x = 0; x < VEC; ++x) {
          if constexpr (SRC == kSrcRows) {
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
      int local = pair, K = A.src_K[0], q0 = A.src_q0[0];
      const float* gs = A.src_gscore[0];
      const float* sc = A.src_score[0];
      const unsigned char* win = A.src_winner[0];
#pragma unroll
      for (int s = 1; s < kMaxSources; ++s) {
        if (s < A.n_src && pair >= A.first[s]) {
          local = pair - A.first[s];
          K = A.src_K[s];
          q0 = A.src_q0[s];
          gs = A.src_gscore[s];
          sc = A.src_score[s];
          win = A.src_winner[s];
        }
      }
      ModelOps<SRC>::coef(gs[local], sc[local], A.p, my_c, c1);
      my_key = q0 + local / K;
      if (A.U > 1) my_key = my_key * A.U + win[local];  // the query row of the branch that won the pair
    } else {
      ModelOps<SRC>::coef(A.gscore[pair], A.score[pair], A.p, my_c, c1);
      my_key = pair / A.K;
      if (A.U > 1) my_key = my_key * A.U + A.winner[pair];
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

// runs in flight per wavefront in the short-segment kernel / the long-segment kernel
constexpr int kRunsShort = 2;
constexpr int kRunsLong = 4;

// Short segments (at most A.short_max pairs).  The sorted pair list is cut into chunks of 64
// positions and a fixed grid of wavefronts strides over the chunks; a wavefront owns the short
// segments that START in its chunk, so its work is bounded by 64 + short_max pairs however the
// segment lengths are distributed.  The lanes fetch the chunk's per-position inputs at once; the
// wavefront then finishes one segment after the other, and while it works on one it already has
// the next one's w, m, v rows on the way (two register sets used in turn).
template <int SRC, int VEC, int NIT, bool REG>
__global__ __launch_bounds__(256) void entity_segment_kernel(EntityArgs A) {
  constexpr int MUL = src_mul(SRC);
  constexpr int R = kRunsShort;
  if (blockIdx.x == 0 && threadIdx.x == 0) *A.fix_count = 0;  // the tile pass, launched after this one, appends to the list
  const int lane = threadIdx.x & 63;
  const int wave = uniform(threadIdx.x >> 6);
  const int n_waves = gridDim.x * 4;
  const int n_chunks = (A.n_pairs + A.chunk - 1) / A.chunk;
  const int n_valid = *A.n_uniq;  // a last segment beyond this one holds the pairs whose id is outside the table: skipped
  if (n_valid < 0) return;  // the plan's build gave up: nothing of it may be read
  const bool mixed = SRC != kSrcRows && A.rows_first < A.n_pairs;  // the plan also holds gradient rows of plain lookups

  for (int chunk = blockIdx.x * 4 + wave; chunk < n_chunks; chunk += n_waves) {
    const int base = chunk * A.chunk;  // the window is 64 positions wide whatever the chunk: a segment that starts in
    const int n_here = min(64, A.n_pairs - base);  // the chunk usually ends inside it
    const int pos = base + min(lane, n_here - 1);
    const int my_seg = A.seg_of_pos[pos];
    const int my_s0 = A.seg_start[my_seg];
    const int my_s1 = A.seg_start[my_seg + 1];
    const int my_len = my_s1 - my_s0;
    bool done_elsewhere = A.skip_single && my_len == 1;  // by the pair-ordered kernel -- unless the one pair is a gradient row
    if (SRC != kSrcRows && mixed && done_elsewhere) done_elsewhere = A.order[pos] < A.rows_first;
    unsigned long long todo = __ballot(lane < n_here && lane < A.chunk && my_s0 == pos && my_len <= A.short_max &&
                                       !done_elsewhere && my_seg < n_valid);
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
      collect_runs<SRC, R>(rs, j, j_end, my_key, my_c);
      request_runs<SRC, VEC, NIT, R>(A, lane, rs, rr);
      if (nxt >= 0) request_state<SRC, VEC, NIT>(A, lane, (unsigned)__builtin_amdgcn_readlane(my_id, nxt), ahead);
      apply_runs<SRC, VEC, NIT, REG, R>(A, rs, rr, cur.e, g1, g2);
      while (j < j_end) {
        collect_runs<SRC, R>(rs, j, j_end, my_key, my_c);
        request_runs<SRC, VEC, NIT, R>(A, lane, rs, rr);
        apply_runs<SRC, VEC, NIT, REG, R>(A, rs, rr, cur.e, g1, g2);
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
template <int SRC, int VEC, int NIT, bool REG>
__global__ __launch_bounds__(256) void entity_tile_kernel(EntityArgs A) {
  constexpr int MUL = src_mul(SRC);
  constexpr int R = kRunsLong;
  const int lane = threadIdx.x & 63;
  const int wave = uniform(threadIdx.x >> 6);
  const int t = blockIdx.x * 4 + wave;
  const int p0 = t * A.tile;
  if (p0 >= A.n_pairs) return;  // whole wavefront leaves; no workgroup barrier is used below
  const int p1 = min(A.n_pairs, p0 + A.tile);
  const int n_valid = *A.n_uniq;  // the segment of ids outside the table, if there is one, is number n_valid: skipped
  if (n_valid < 0) return;  // the plan's build gave up: nothing of it may be read
  const bool mixed = SRC != kSrcRows && A.rows_first < A.n_pairs;  // the plan also holds gradient rows of plain lookups
  {  // does a long segment that came in from the left end inside this tile?  The fix-up pass finishes it.
    const int sg = A.seg_of_pos[p0];
    const int b0 = A.seg_start[sg], b1 = A.seg_start[sg + 1];
    if (lane == 0 && p0 > 0 && b0 < p0 && b1 <= p1 && b1 - b0 > A.short_max && sg < n_valid)
      A.fix_list[atomicAdd(A.fix_count, 1)] = t;
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
      } else if (SRC != kSrcRows) {
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
          collect_runs<SRC, R>(rs, j, j_end, my_key, my_c);
          request_runs<SRC, VEC, NIT, R>(A, lane, rs, rr);
          apply_runs<SRC, VEC, NIT, REG, R>(A, rs, rr, st.e, g1, g2);
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

// The tiles whose first segment is long, came in from the left and ends inside the tile are on the list the
// tile pass made; a fixed grid of workgroups takes them in turn.  For each, the workgroup adds that segment's
// partial rows (tails of the tiles it crossed, then this tile's head) in tile order and finishes the row.
// The order of the list (the tile pass appends with an integer atomic) decides who does what, not any result.
template <int SRC, int VEC, int NIT, int NW, bool REG>
__global__ __launch_bounds__(NW * 64) void entity_fixup_kernel(EntityArgs A) {
  constexpr int MUL = src_mul(SRC);
  extern __shared__ float lds[];
  const int lane = threadIdx.x & 63;
  const int wave = uniform(threadIdx.x >> 6);
  const int half = A.ncol * VEC;
  const size_t row_len = (size_t)half * MUL;
  const int n_fix = *A.fix_count;
  const bool mixed = SRC != kSrcRows && A.rows_first < A.n_pairs;
  for (int item = blockIdx.x; item < n_fix; item += gridDim.x) {  // uniform over the workgroup
  const int t = A.fix_list[item];
  const int p0 = t * A.tile;
  const int seg = A.seg_of_pos[p0];
  const int s0 = A.seg_start[seg];
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
  __syncthreads();  // the LDS rows are free again for the workgroup's next item
  }
}

// ---- sign-coded sources (box, L1) ---------------------------------------------------------------
// The gradient of a run is +-c per feature, the choice being the run's code bytes (64 * NIT per pair, written by
// the forward).  Nothing else is read per run, so these kernels are a chain of dependent gathers -- sorted
// position -> pair -> upstream gradient and code bytes -- and what bounds them is how many of those a wavefront
// keeps in flight.  Both kernels therefore fetch per window of 64 sorted positions, one position per lane: all
// lanes gather their pair's upstream gradient at once, then every lane that starts a run loads that run's
// whole code record (64 * NIT contiguous bytes, one memory sector or two) and parks it in the wavefront's
// LDS slab; the runs are then summed from LDS (lane l reads byte l of the run's record).  One memory latency
// per step of the chain and window, instead of one per handful of runs.
constexpr int kTile = 256;      // sorted positions per tile of the long-segment pass
constexpr int kShortMax = 64;   // longest segment one wavefront finishes on its own
constexpr int kTileWindows = kTile / 64;

typedef unsigned code_vec4 __attribute__((ext_vector_type(4)));

struct CodedLane {
  int key;     // query number of the lane's pair (-1: the lane holds no pair that matters)
  float c;     // its coefficient
  int pair;    // >= 0: a model pair; < 0: ~(row number) of a gradient row of a plain lookup
  const unsigned char* code;  // the pair's code record
};

// What the lane needs to know about plan pair `plan_pair` (the value of order[] at its position).
template <int SRC, int NIT>
__device__ __forceinline__ CodedLane resolve_coded_lane(const EntityArgs& A, int plan_pair, bool want) {
  CodedLane L{-1, 0.f, 0, A.codes};
  if (!want) return L;
  const bool is_row = plan_pair >= A.rows_first;
  const int pair = is_row ? 0 : plan_pair;  // a pair whose inputs exist
  int local = pair, K = A.K, q0 = 0;
  const float* gs = A.gscore;
  const float* sc = A.score;
  const unsigned char* cb = A.codes;
  if (A.n_src > 1) {  // uniform: which index stream the pair came from, and its number inside that stream
    K = A.src_K[0];
    q0 = A.src_q0[0];
    gs = A.src_gscore[0];
    sc = A.src_score[0];
    cb = A.src_codes[0];
#pragma unroll
    for (int s = 1; s < kMaxSources; ++s) {
      if (s < A.n_src && pair >= A.first[s]) {
        local = pair - A.first[s];
        K = A.src_K[s];
        q0 = A.src_q0[s];
        gs = A.src_gscore[s];
        sc = A.src_score[s];
        cb = A.src_codes[s];
      }
    }
  }
  float c1;
  ModelOps<SRC>::coef(gs[local], sc[local], A.p, L.c, c1);
  L.key = q0 + local / K;
  L.pair = pair;
  L.code = cb + (size_t)local * (NIT * 64);
  if (is_row) {
    L.c = 0.f;
    L.key = -2;
    L.pair = ~(plan_pair - A.rows_first);
  }
  return L;
}

// Lanes that start a run: the first lane, or another query or another entity than the lane before.  Gradient
// rows start none.
__device__ __forceinline__ bool starts_run(int lane, const CodedLane& L, unsigned id) {
  const int prev_key = __shfl_up(L.key, 1);
  const unsigned prev_id = (unsigned)__shfl_up((int)id, 1);
  return L.key >= 0 && (lane == 0 || prev_key != L.key || prev_id != id);
}

template <int NIT>
__device__ __forceinline__ void request_code_record(code_vec4 (&cd)[NIT * 4], const CodedLane& L, bool head) {
#pragma unroll
  for (int i = 0; i < NIT * 4; ++i) cd[i] = code_vec4{0u, 0u, 0u, 0u};
  if (head) {
#pragma unroll
    for (int i = 0; i < NIT * 4; ++i) cd[i] = reinterpret_cast<const code_vec4*>(L.code)[i];
  }
}

// Orders a wavefront's own LDS writes before its later LDS reads (other lanes' entries).
__device__ __forceinline__ void entity_slab_fence() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

template <int NIT>
__device__ __forceinline__ void park_code_records(unsigned char* slab, int lane, const code_vec4 (&cd)[NIT * 4], bool head) {
  entity_slab_fence();  // reads of the previous window are done
  if (head) {
#pragma unroll
    for (int i = 0; i < NIT * 4; ++i) reinterpret_cast<code_vec4*>(slab + lane * (NIT * 64))[i] = cd[i];
  }
  entity_slab_fence();
}

// g += the gradient of the runs that lanes [j, j_end) of the window hold, in lane order: the coefficients of a
// run are summed first (lane order), then the run's +-c terms are added; R runs' code bytes are read from
// the slab before the first is used.
template <int SRC, int VEC, int NIT, int R = 8>
__device__ __forceinline__ void add_coded_runs(const EntityArgs& A, const unsigned char* slab, int lane, int j, int j_end,
                                               int my_key, float my_c, float (&g1)[NIT][VEC]) {
  while (j < j_end) {
    int head[R], n = 0;
    float c[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      head[r] = 0;
      c[r] = 0.f;
      if (j < j_end) {  // wave-uniform
        n = r + 1;
        head[r] = j;
        const int key = __builtin_amdgcn_readlane(my_key, j);
        do {
          c[r] += __int_as_float(__builtin_amdgcn_readlane(__float_as_int(my_c), j));
          ++j;
        } while (j < j_end && __builtin_amdgcn_readlane(my_key, j) == key);
      }
    }
    unsigned code[R][NIT];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      if (r < n) {
#pragma unroll
        for (int it = 0; it < NIT; ++it) code[r][it] = slab[head[r] * (NIT * 64) + 64 * it + lane];
      }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      if (r < n) {
#pragma unroll
        for (int it = 0; it < NIT; ++it)
#pragma unroll
          for (int x = 0; x < VEC; ++x)
            ModelOps<SRC>::bwd_e_coded(c[r], second_coef<SRC>(c[r], A.p), code[r][it], VEC - 1 - x, g1[it][x]);
      }
    }
  }
}

// Short segments, as entity_segment_kernel: chunks of 64 sorted positions, a wavefront finishes the short
// segments that start in its chunk.  The chunk's gathers are made once for all of them (only by the lanes of those
// segments), and the w, m, v rows of up to S segments are requested before the first is finished.
template <int SRC, int VEC, int NIT>
__global__ __launch_bounds__(256) void entity_segment_coded_kernel(EntityArgs A) {
  static_assert(src_mul(SRC) == 1, "sign codes exist for one-half rows");
  constexpr int S = NIT == 1 ? 4 : 2;
  extern __shared__ unsigned char code_lds[];  // [4 wavefronts][64 records]
  if (blockIdx.x == 0 && threadIdx.x == 0) *A.fix_count = 0;  // the tile pass, launched after this one, appends to the list
  const int lane = threadIdx.x & 63;
  const int wave = uniform(threadIdx.x >> 6);
  unsigned char* slab = code_lds + wave * (64 * NIT * 64);
  const int n_waves = gridDim.x * 4;
  const int n_chunks = (A.n_pairs + A.chunk - 1) / A.chunk;
  const int n_valid = *A.n_uniq;  // a last segment beyond this one holds the pairs whose id is outside the table: skipped
  if (n_valid < 0) return;  // the plan's build gave up: nothing of it may be read
  const bool mixed = A.rows_first < A.n_pairs;  // the plan also holds gradient rows of plain lookups

  for (int chunk = blockIdx.x * 4 + wave; chunk < n_chunks; chunk += n_waves) {
    const int base = chunk * A.chunk;  // the window is 64 positions wide whatever the chunk: a segment that starts in
    const int n_here = min(64, A.n_pairs - base);  // the chunk usually ends inside it
    const int pos = base + min(lane, n_here - 1);
    const int my_seg = A.seg_of_pos[pos];
    const int my_plan_pair = A.order[pos];
    const unsigned my_id = (unsigned)A.sorted_ids[pos];
    const int my_s0 = A.seg_start[my_seg];
    const int my_s1 = A.seg_start[my_seg + 1];
    const int my_len = my_s1 - my_s0;
    // a one-pair segment was finished by the pair-ordered kernel -- unless its one pair is a gradient row
    const bool done_elsewhere = A.skip_single && my_len == 1 && !(mixed && my_plan_pair >= A.rows_first);
    const bool mine = lane < n_here && my_len <= A.short_max && !done_elsewhere && my_seg < n_valid;
    unsigned long long todo = __ballot(mine && my_s0 == pos && lane < A.chunk);
    if (todo == 0ull) continue;

    int win_base = base;
    unsigned win_id = my_id;
    // the lanes of segments that started before the chunk belong to another wavefront's work
    CodedLane cur = resolve_coded_lane<SRC, NIT>(A, my_plan_pair, mine && my_s0 >= base && my_s0 < base + A.chunk);
    {
      const bool head = starts_run(lane, cur, win_id);
      code_vec4 cd[NIT * 4];
      request_code_record<NIT>(cd, cur, head);
      park_code_records<NIT>(slab, lane, cd, head);
    }
    // a segment that runs past the window: the window restarts at its first pair (every lane fetches)
    auto restart_window = [&](int s0) {
      win_base = s0;
      const int q = min(s0 + lane, A.n_pairs - 1);
      const bool in = s0 + lane < A.n_pairs;
      win_id = (unsigned)A.sorted_ids[q];
      cur = resolve_coded_lane<SRC, NIT>(A, A.order[q], in);
      const bool head = starts_run(lane, cur, win_id);
      code_vec4 cd[NIT * 4];
      request_code_record<NIT>(cd, cur, head);
      park_code_records<NIT>(slab, lane, cd, head);
    };

    while (todo != 0ull) {
      int at[S];
      RowState<1, VEC, NIT> st[S];
#pragma unroll
      for (int s = 0; s < S; ++s) {
        at[s] = todo != 0ull ? __builtin_ctzll(todo) : -1;
        if (at[s] >= 0) {  // wave-uniform
          todo &= todo - 1;
          request_state<SRC, VEC, NIT>(A, lane, (unsigned)__builtin_amdgcn_readlane((int)my_id, at[s]), st[s]);
        }
      }
#pragma unroll
      for (int s = 0; s < S; ++s) {
        if (at[s] >= 0) {
          const int i = at[s];
          const int s0 = base + i;
          const int s1 = __builtin_amdgcn_readlane(my_s1, i);
          const unsigned row_id = (unsigned)__builtin_amdgcn_readlane((int)my_id, i);
          const int seg = __builtin_amdgcn_readlane(my_seg, i);
          if (s1 > win_base + 64) restart_window(s0);
          float g1[NIT][VEC], g2[NIT][VEC];
          zero_acc<VEC, NIT>(g1, g2);
          const int j = s0 - win_base;
          const int j_all = s1 - win_base;
          const int j_end = mixed ? j_all - rows_in_window(cur.pair, j, j_all) : j_all;  // the model's pairs come first
          add_coded_runs<SRC, VEC, NIT>(A, slab, lane, j, j_end, cur.key, cur.c, g1);
          auto grad_rows_of_segment = [&](float (&a1)[NIT][VEC], float (&a2)[NIT][VEC]) {
            if (j_end < j_all) add_grad_rows<1, VEC, NIT>(A, lane, ~cur.pair, j_end, j_all, a1, a2);  // plain lookups only
          };
          finish_row<SRC, VEC, NIT, false>(A, lane, row_id, seg, g1, g2, st[s].e, st[s].m, st[s].v, grad_rows_of_segment);
        }
      }
    }
  }
}

// Long segments, as entity_tile_kernel: one wavefront per tile of 256 sorted positions.  The tile's segment
// numbers, bounds and ids are fetched once (four positions per lane) and every later question about them is
// answered from those registers; the stretch of a long segment inside the tile has its windows' gathers issued
// together (W windows at a time), so the chain position -> pair -> upstream gradient / code record costs three
// memory latencies per stretch.
template <int SRC, int VEC, int NIT>
__global__ __launch_bounds__(256, 4) void entity_tile_coded_kernel(EntityArgs A) {
  static_assert(src_mul(SRC) == 1, "sign codes exist for one-half rows");
  constexpr int TW = kTileWindows;
  constexpr int W = NIT == 1 ? 4 : 2;  // windows whose code records are in registers at a time
  extern __shared__ unsigned char code_lds[];  // [4 wavefronts][64 records]
  const int lane = threadIdx.x & 63;
  const int wave = uniform(threadIdx.x >> 6);
  unsigned char* slab = code_lds + wave * (64 * NIT * 64);
  const int t = blockIdx.x * 4 + wave;
  const int p0 = t * kTile;
  if (p0 >= A.n_pairs) return;  // whole wavefront leaves; no workgroup barrier is used below
  const int p1 = min(A.n_pairs, p0 + kTile);
  const int n_valid = *A.n_uniq;  // the segment of ids outside the table, if there is one, is number n_valid: skipped
  if (n_valid < 0) return;  // the plan's build gave up: nothing of it may be read
  const bool mixed = A.rows_first < A.n_pairs;

  int sg[TW], b0[TW], b1[TW], id[TW];
#pragma unroll
  for (int w = 0; w < TW; ++w) {
    const int q = min(p0 + 64 * w + lane, p1 - 1);
    sg[w] = A.seg_of_pos[q];
    id[w] = A.sorted_ids[q];
  }
#pragma unroll
  for (int w = 0; w < TW; ++w) {
    b0[w] = A.seg_start[sg[w]];
    b1[w] = A.seg_start[sg[w] + 1];
  }
  // what position p0 + rel of the tile says (read out of all four registers, then chosen: scalar work)
  auto at = [&](const int (&v)[TW], int rel) {
    const int w = rel >> 6, l = rel & 63;
    int x = __builtin_amdgcn_readlane(v[0], l);
#pragma unroll
    for (int u = 1; u < TW; ++u) {
      const int y = __builtin_amdgcn_readlane(v[u], l);
      x = w == u ? y : x;
    }
    return x;
  };
  {  // does a long segment that came in from the left end inside this tile?  The fix-up pass finishes it.
    const int s = at(sg, 0), s0 = at(b0, 0), s1 = at(b1, 0);
    if (lane == 0 && p0 > 0 && s0 < p0 && s1 <= p1 && s1 - s0 > A.short_max && s < n_valid)
      A.fix_list[atomicAdd(A.fix_count, 1)] = t;
  }
  bool any_long = false;
#pragma unroll
  for (int w = 0; w < TW; ++w)
    any_long |= __ballot(p0 + 64 * w + lane < p1 && b1[w] - b0[w] > A.short_max && sg[w] < n_valid) != 0ull;
  if (!any_long) return;  // most tiles hold short segments only

  int pos = p0;
  while (pos < p1) {
    const int rel = pos - p0;
    const int seg = at(sg, rel), s0 = at(b0, rel), s1 = at(b1, rel);
    const int end = min(s1, p1);
    if (s1 - s0 > A.short_max && seg < n_valid) {
      const unsigned row_id = (unsigned)at(id, rel);
      const bool whole = s0 >= p0 && s1 <= p1;
      RowState<1, VEC, NIT> st;
      if (whole) request_state<SRC, VEC, NIT>(A, lane, row_id, st);
      float g1[NIT][VEC], g2[NIT][VEC];
      zero_acc<VEC, NIT>(g1, g2);
      for (int gbase = pos; gbase < end; gbase += 64 * W) {  // uniform
        int pp[W];
#pragma unroll
        for (int w = 0; w < W; ++w) {
          const int base = gbase + 64 * w;
          pp[w] = base < end ? A.order[min(base + lane, end - 1)] : 0;
        }
        CodedLane L[W];
#pragma unroll
        for (int w = 0; w < W; ++w) {
          const int base = gbase + 64 * w;
          L[w] = resolve_coded_lane<SRC, NIT>(A, pp[w], base + lane < end);
        }
        code_vec4 cd[W][NIT * 4];
        unsigned long long heads[W];
#pragma unroll
        for (int w = 0; w < W; ++w) {
          const bool head = starts_run(lane, L[w], row_id);  // one entity: a run ends where the query changes
          heads[w] = __ballot(head);
          request_code_record<NIT>(cd[w], L[w], head);
        }
#pragma unroll
        for (int w = 0; w < W; ++w) {
          const int base = gbase + 64 * w;
          if (base < end) {  // uniform
            park_code_records<NIT>(slab, lane, cd[w], (heads[w] >> lane) & 1ull);
            int j_end = min(64, end - base);
            if (mixed) j_end -= rows_in_window(L[w].pair, 0, j_end);  // gradient rows wait for the row's finish
            add_coded_runs<SRC, VEC, NIT>(A, slab, lane, 0, j_end, L[w].key, L[w].c, g1);
          }
        }
      }
      if (whole) {
        auto grad_rows_of_segment = [&](float (&a1)[NIT][VEC], float (&a2)[NIT][VEC]) {
          if (mixed)
            add_segment_grad_rows<1, VEC, NIT>(A, lane, first_grad_row_of_segment(A, lane, s0, s1), s1, 0, 1, a1, a2);
        };
        finish_row<SRC, VEC, NIT, false>(A, lane, row_id, seg, g1, g2, st.e, st.m, st.v, grad_rows_of_segment);
      } else if (s1 > p1)
        store_partial<SRC, VEC, NIT>(A, A.tail, t, lane, g1, g2);
      else
        store_partial<SRC, VEC, NIT>(A, A.head, t, lane, g1, g2);
    }
    pos = end;
  }
}

// Workgroups of 256 threads of `kernel` (with that much dynamic LDS) the current device keeps resident; asked
// once per kernel and device.
template <class K>
unsigned resident_blocks(K kernel, int dynamic_lds) {
  static std::mutex mu;
  static std::map<std::pair<const void*, int>, unsigned> cached;  // (kernel, device) -> workgroups
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 256u * 8u;
  const std::pair<const void*, int> key(reinterpret_cast<const void*>(kernel), dev);
  std::lock_guard<std::mutex> lock(mu);
  auto it = cached.find(key);
  if (it != cached.end()) return it->second;
  int cus = 0, per_cu = 0;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
      hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, 256, dynamic_lds) != hipSuccess || cus <= 0 || per_cu <= 0)
    return 256u * 8u;
  return cached[key] = (unsigned)cus * (unsigned)per_cu;
}

template <int SRC, int VEC, int NIT, bool REG>
int launch_entity_reg(hipStream_t st, const EntityArgs& A) {
  const unsigned tiles = (unsigned)((A.n_pairs + A.tile - 1) / A.tile);
  // short segments: a fixed grid of wavefronts strides over the segment list (its length lives on the device)
  // (as many workgroups as the chip holds at once: a second wave of workgroups would run half empty)
  const unsigned want_blocks = (unsigned)(((A.n_pairs + A.chunk - 1) / A.chunk + 3) / 4);
  bool coded = false;
  // (sign codes exist for rows of up to two column groups)
  if constexpr (SRC != kSrcRows && model_coded(SRC) && !REG && NIT <= 2) coded = A.codes != nullptr;
  if (coded) {
    if constexpr (SRC != kSrcRows && model_coded(SRC) && !REG && NIT <= 2) {
      const size_t slabs = (size_t)4 * 64 * NIT * 64;  // one code record per lane and wavefront
      const unsigned seg_blocks =
          min(want_blocks, resident_blocks(entity_segment_coded_kernel<SRC, VEC, NIT>, (int)slabs));
      hipLaunchKernelGGL((entity_segment_coded_kernel<SRC, VEC, NIT>), dim3(seg_blocks), dim3(256), slabs, st, A);
      hipLaunchKernelGGL((entity_tile_coded_kernel<SRC, VEC, NIT>), dim3((tiles + 3) / 4), dim3(256), slabs, st, A);
    }
  } else {
    const unsigned seg_blocks = min(want_blocks, resident_blocks(entity_segment_kernel<SRC, VEC, NIT, REG>, 0));
    hipLaunchKernelGGL((entity_segment_kernel<SRC, VEC, NIT, REG>), dim3(seg_blocks), dim3(256), 0, st, A);
    hipLaunchKernelGGL((entity_tile_kernel<SRC, VEC, NIT, REG>), dim3((tiles + 3) / 4), dim3(256), 0, st, A);
  }
  const size_t row_bytes = (size_t)A.ncol * VEC * src_mul(SRC) * sizeof(float);
  const bool mixed = SRC != kSrcRows && A.rows_first < A.n_pairs;
  // the fix-up pass: a fixed grid takes the listed tiles in turn (at most one per tile; usually far fewer)
  const unsigned fix_blocks = min(tiles, 1024u);
  EntityArgs F = A;
  if (7 * row_bytes <= 60 * 1024) {
    F.share_rows = mixed && 14 * row_bytes <= 60 * 1024;
    hipLaunchKernelGGL((entity_fixup_kernel<SRC, VEC, NIT, 8, REG>), dim3(fix_blocks), dim3(8 * 64),
                       (F.share_rows ? 14 : 7) * row_bytes, st, F);
  } else {
    F.share_rows = mixed && 6 * row_bytes <= 60 * 1024;
    hipLaunchKernelGGL((entity_fixup_kernel<SRC, VEC, NIT, 4, REG>), dim3(fix_blocks), dim3(4 * 64),
                       (F.share_rows ? 6 : 3) * row_bytes, st, F);
  }
  return check_launch("entity backward");
}

template <int SRC, int VEC, int NIT>
int launch_entity(hipStream_t st, const EntityArgs& A) {
  if constexpr (SRC == mBetaKL || SRC == mComplex || SRC == mDistmult) {
    if (SRC == mBetaKL ? A.p.reg_on : A.p.norm_on) return launch_entity_reg<SRC, VEC, NIT, true>(st, A);
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
