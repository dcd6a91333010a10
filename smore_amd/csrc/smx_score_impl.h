// Gather-fused scoring, forward and query-side backward (fp32).
//
// Replaces, in one pass each, the sequence the reference runs per training
// step for the negative samples (smore/models/kg_reasoning.py:301-307,349-355):
//   rows = table[idx]                      smore/common/embedding/embed_rw.py:74-75
//   [optional clamp(rows + 1, .05, 1e9)]   smore/common/modules.py:29-36
//   d = dist(rows, query)                  smore/common/torchext/common_kernel.h:33-56
//   logit = gamma - d                      custom_cal_logit of smore/models/*.py
// and, backward, the query-gradient kernel common_kernel.h:92-123.  The
// [B,K,D] gathered tensor is never materialised: a wavefront reads each entity
// row straight from the table with 16-byte loads (one float4 column per lane).
//
// Work split.  forward: workgroup = (query b, tile of negatives); the query
// row(s) are staged once in LDS, every lane then keeps the features it owns in
// registers for the whole tile; each of the four wavefronts streams its
// quarter of the tile's rows, two batches of rows in flight at a time.  backward: one workgroup per
// query walks all K negatives, wavefront partial sums are combined through LDS
// in wavefront order, so the gradient has a fixed summation order.
#pragma once
#include "smx_common.h"
#include "smx_models.h"
#include "smx_rowupdate.h"
#include "smx_wave.h"

namespace smx {

struct ScoreArgs {
  const float* table;
  const long long* idx;  // null: `table` holds the B*K rows in pair order
  const float* q1;
  const float* q2;
  float* score_out;      // forward
  const float* score;    // backward: the logits the forward wrote
  const float* gscore;
  float* gq1;
  float* gq2;
  int B, K, ncol;
  int ids_shared;        // idx holds K ids that every query scores (--share_negative, online_sampler.py:155-157), not B*K
  // Union queries (kg_reasoning.py:326, box.py:163): q1 / q2 hold U branch rows per query, [B*U, dim]; a kernel's
  // "query" is then one branch row, number bq = b * U + u, which scores the ids of query b.
  int U;                 // branches per query (1: none of this)
  const unsigned char* winner;  // query backward, [B, K]: the branch that gave the pair's logit; a branch row sums its own pairs only
  unsigned long long n_rows;
  ScoreParams p;
  int* err;
  const int* pair_seg;   // one-pair segments finished by the query backward (SINGLES kernels)
  const long long* uniq; // plan's id list: row of a one-pair segment when the kernel runs without the id tensor (GQ = false)
  unsigned char* codes;  // [B*K][NIT*64] sign codes written by this kernel (forward or query backward), or null
  const unsigned char* codes_in;  // query backward: codes the forward left; the entity rows are then not read
  RowSink sink;
};

template <int VEC> struct Pack {
  float v[VEC];
};

template <int VEC>
__device__ __forceinline__ Pack<VEC> load_pack(const float* __restrict__ base, int col) {
  Pack<VEC> r;
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

// Loads the features a lane owns of the staged query into registers.
template <int M, int VEC, int NIT, bool FWD>
__device__ __forceinline__ void load_query_regs(const float* lds, int dim, int ncol, int lane,
                                                typename ModelOps<M>::Q (&q)[NIT][VEC]) {
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    const int c = lane + 64 * it;
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      const int cc = min(c, ncol - 1);  // lanes past the row end hold a copy of the last column
      const float a = lds[cc * VEC + v];
      const float b = model_nq(M) == 2 ? lds[dim + cc * VEC + v] : 0.f;
      q[it][v] = FWD ? prep_forward<M>(a, b) : prep_backward_query<M>(a, b);
    }
  }
}

template <int M>
__device__ __forceinline__ void stage_query(float* lds, const float* __restrict__ q1, const float* __restrict__ q2,
                                            size_t b, int dim) {
  for (int d = threadIdx.x; d < dim; d += blockDim.x) {
    lds[d] = q1[b * dim + d];
    if (model_nq(M) == 2) lds[dim + d] = q2[b * dim + d];
  }
  __syncthreads();
}

// ---- streaming the rows of up to 64 pairs through a wavefront -----------------------------------
// The lanes first fetch, in one coalesced load, the ids of the pairs the wavefront is about to
// process (pair j of the batch lives in lane j), turn them into row addresses and park them, with the
// pair's two gradient coefficients in the backward kernel, in a 64-entry slab of LDS that belongs to
// the wavefront.  The row loop then finds a row with one LDS read at a uniform address (a broadcast,
// no bank conflicts) instead of v_readlane + scalar address arithmetic per row: the loop is bound by
// instruction issue, and every vector or scalar instruction it does not need is time.  Rows are
// requested RIF at a time into two register sets used in turn: while set A is consumed, set B is
// already on its way.  All loads are unconditional so that they issue as one batch and stay in
// flight together: entries past the batch's end repeat its last pair.

struct PairBatch {
  unsigned off_lo, off_hi;  // this lane's pair: offset of its entity row in floats
  unsigned row;             // ... and the row number (low 32 bits)
};

__device__ __forceinline__ PairBatch load_pair_batch(const long long* __restrict__ idx, size_t first_pair, int cnt,
                                                     int lane, size_t row_len, unsigned long long n_rows, int& bad) {
  const size_t pair = first_pair + min(lane, cnt - 1);
  long long row = idx ? idx[pair] : (long long)pair;
  if ((unsigned long long)row >= n_rows) {  // id outside the table: remember it, read row 0 instead
    bad = 1;
    row = 0;
  }
  const unsigned long long off = (unsigned long long)row * row_len;
  return {(unsigned)off, (unsigned)(off >> 32), (unsigned)row};
}

__device__ __forceinline__ unsigned long long batch_off(const PairBatch& pb, int j) {
  const unsigned lo = (unsigned)__builtin_amdgcn_readlane((int)pb.off_lo, j);
  const unsigned hi = (unsigned)__builtin_amdgcn_readlane((int)pb.off_hi, j);
  return ((unsigned long long)hi << 32) | lo;
}

constexpr int kSlabDwords = 64 * 4;  // per wavefront: 64 entries of {address lo, address hi, c0, c1}

// Orders a wavefront's own LDS writes before its later LDS reads (other lanes' entries).
__device__ __forceinline__ void slab_fence() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

__device__ __forceinline__ void stage_pairs(unsigned* slab, int lane, const float* __restrict__ table,
                                            const PairBatch& pb, float c0, float c1) {
  slab_fence();  // reads of the previous batch are done
  const unsigned long long addr =
      (unsigned long long)(table + (((unsigned long long)pb.off_hi << 32) | pb.off_lo));
  *reinterpret_cast<uint4*>(slab + 4 * lane) =
      make_uint4((unsigned)addr, (unsigned)(addr >> 32), __float_as_uint(c0), __float_as_uint(c1));
  slab_fence();
}

// The address comes back from LDS as an integer; the pointer made from it is declared global so that
// the row loads are global_load (a generic pointer would make them flat_load, which also counts
// against the LDS wait counter).
typedef const __attribute__((address_space(1))) float* GlobalRow;
__device__ __forceinline__ GlobalRow slab_row(const unsigned* slab, int j) {
  const uint2 a = *reinterpret_cast<const uint2*>(slab + 4 * j);
  return reinterpret_cast<GlobalRow>(((unsigned long long)a.y << 32) | a.x);
}
template <int VEC>
__device__ __forceinline__ Pack<VEC> load_pack(GlobalRow base, int col) {
  Pack<VEC> r;
  if constexpr (VEC == 4) {
    typedef float vec4 __attribute__((ext_vector_type(4)));
    const vec4 t = reinterpret_cast<const __attribute__((address_space(1))) vec4*>(base)[col];
    r.v[0] = t.x;
    r.v[1] = t.y;
    r.v[2] = t.z;
    r.v[3] = t.w;
  } else {
    r.v[0] = base[col];
  }
  return r;
}
__device__ __forceinline__ float2 slab_coef(const unsigned* slab, int j) {
  return *reinterpret_cast<const float2*>(slab + 4 * j + 2);
}

template <int MUL, int VEC, int NIT, int RIF> struct RowSet {
  Pack<VEC> e1[RIF][NIT];
  Pack<VEC> e2[RIF][NIT];
};

// Requests rows g0 .. g0+RIF-1 of the batch; g0 is a multiple of RIF, so the entries exist.
template <int MUL, int VEC, int NIT, int RIF>
__device__ __forceinline__ void request_rows(RowSet<MUL, VEC, NIT, RIF>& rs, const unsigned* slab, int g0, int dim,
                                             int ncol, int lane) {
  GlobalRow pe[RIF];
#pragma unroll
  for (int r = 0; r < RIF; ++r) pe[r] = slab_row(slab, g0 + r);
#pragma unroll
  for (int r = 0; r < RIF; ++r) {
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      const int c = min(lane + 64 * it, ncol - 1);
      rs.e1[r][it] = load_pack<VEC>(pe[r], c);
      if (MUL == 2) rs.e2[r][it] = load_pack<VEC>(pe[r] + dim, c);
    }
    // Rows are used in the order r = 0, 1, ..: their loads must be issued in that order everywhere (the
    // scheduler is otherwise free to reverse them in the loop prologue), or the wait for row 0 at the top
    // of the streaming loop becomes a wait for every load in flight.
    __builtin_amdgcn_sched_barrier(0);
  }
}

// Streams the cnt (<= 64) rows of a staged batch through `consume(j, e1, e2)`, j ascending.
template <int MUL, int VEC, int NIT, int RIF, class Consume>
__device__ __forceinline__ void stream_batch(const unsigned* slab, int cnt, int dim, int ncol, int lane,
                                             Consume&& consume) {
  static_assert(64 % RIF == 0, "a group of rows must not straddle the end of the slab");
  RowSet<MUL, VEC, NIT, RIF> a, b;
  const int last = ((cnt - 1) / RIF) * RIF;  // first row of the last group
  request_rows<MUL, VEC, NIT, RIF>(a, slab, 0, dim, ncol, lane);
  for (int j0 = 0; j0 < cnt; j0 += 2 * RIF) {
    request_rows<MUL, VEC, NIT, RIF>(b, slab, min(j0 + RIF, last), dim, ncol, lane);
#pragma unroll
    for (int r = 0; r < RIF; ++r)
      if (j0 + r < cnt) consume(j0 + r, a.e1[r], a.e2[r]);
    request_rows<MUL, VEC, NIT, RIF>(a, slab, min(j0 + 2 * RIF, last), dim, ncol, lane);
#pragma unroll
    for (int r = 0; r < RIF; ++r)
      if (j0 + RIF + r < cnt) consume(j0 + RIF + r, b.e1[r], b.e2[r]);
  }
}

// Sign codes on their way to memory: a wavefront parks each pair's NIT x 64 code bytes in its LDS
// stage and, every 16 pairs (and after the last one), writes the stage out with 16-byte stores -- the
// 16 pairs are contiguous in the code array as well.
constexpr int kStagePairs = 16;
template <int NIT>
__device__ __forceinline__ void flush_codes(const unsigned char* stage, unsigned char* codes, size_t first_pair, int j,
                                            int cnt, int lane) {
  if ((j & (kStagePairs - 1)) == kStagePairs - 1 || j == cnt - 1) {
    slab_fence();
    typedef unsigned vec4u __attribute__((ext_vector_type(4)));
    const int rows_here = (j & (kStagePairs - 1)) + 1;
    vec4u* out = reinterpret_cast<vec4u*>(codes + (first_pair + (j & ~(kStagePairs - 1))) * (size_t)(NIT * 64));
#pragma unroll
    for (int i = 0; i < NIT; ++i) {
      const int chunk = lane + 64 * i;
      if (chunk * 16 < rows_here * NIT * 64)
        __builtin_nontemporal_store(reinterpret_cast<const vec4u*>(stage)[chunk], out + chunk);
    }
    slab_fence();
  }
}

// DEDUP: a workgroup scores each DISTINCT entity among the (up to 256) pairs of its tile once.  With skewed ids a
// query's negatives repeat the hot entities many times (Zipf 1.1: ~175 distinct among 256 consecutive negatives,
// ~51 among 64), every repeat costs the same instructions as the first occurrence although its row comes from
// the cache, and at such shapes the kernel is bound by instruction issue.  The lanes enter their ids into a small
// hash table in LDS; the first pair of the tile with an id puts its row on the tile's list of representatives; the
// list (in pair order) is dealt out to the four wavefronts in equal parts and streamed; every pair then takes its
// score (and its code bytes, from the tile's LDS stage) from its representative: the same bits as without
// de-duplication, pair by pair.
constexpr int kDedupSlots = 512;   // hash table entries for the 256 ids of a tile
constexpr unsigned kDedupEmpty = 0xffffffffu;  // (no id: the table has at most 2^32 - 1 rows)
// LDS bytes of the de-duplication tables: ids, first pairs and list positions of the slots, row addresses and
// scores of the list, representatives per wavefront
constexpr size_t kDedupLds = kDedupSlots * 12 + 256 * 8 + 256 * 4 + 16;

template <int M, int VEC, int NIT, int RIF, bool REG, bool CODED = false, bool DEDUP = false>
__global__ __launch_bounds__(256) void score_forward_kernel(ScoreArgs A, int tiles, int tile_k) {
  const float* __restrict__ table = A.table;
  const long long* __restrict__ idx = A.idx;
  const float* __restrict__ q1 = A.q1;
  const float* __restrict__ q2 = A.q2;
  float* __restrict__ score = A.score_out;
  const int K = A.K, ncol = A.ncol;
  const unsigned long long n_rows = A.n_rows;
  const ScoreParams p = A.p;
  int* err = A.err;
  constexpr int MUL = model_mul(M);
  extern __shared__ float lds[];
  const int b = blockIdx.x / tiles;
  const int tile = blockIdx.x - b * tiles;
  const int lane = threadIdx.x & 63;
  const int wave = uniform(threadIdx.x >> 6);
  const int dim = ncol * VEC;
  const size_t row_len = (size_t)dim * MUL;

  // this wavefront's share of the tile: per_wave (<= 64) consecutive negatives
  const int per_wave = tile_k / 4;
  const int kw0 = tile * tile_k + wave * per_wave;
  const int cnt = min(per_wave, K - kw0);
  int bad = 0;
  PairBatch pb{0u, 0u};
  if (cnt > 0)
    pb = load_pair_batch(idx, (A.ids_shared ? (size_t)0 : (size_t)(b / A.U) * K) + kw0, cnt, lane, row_len, n_rows, bad);

  // LDS: query | per-wavefront pair slabs | code stage (per wavefront; one for the tile with DEDUP) | DEDUP tables
  unsigned* slab = reinterpret_cast<unsigned*>(lds + model_nq(M) * dim) + wave * kSlabDwords;
  constexpr int kStaged = DEDUP ? 256 : kStagePairs;  // pairs whose code bytes a stage holds
  unsigned char* stage_base = reinterpret_cast<unsigned char*>(lds + model_nq(M) * dim + 4 * kSlabDwords);
  unsigned char* stage = DEDUP ? stage_base : stage_base + wave * (kStaged * NIT * 64);
  unsigned char* after_stage = stage_base + (CODED ? (size_t)(DEDUP ? 1 : 4) * kStaged * NIT * 64 : 0);
  unsigned* slot_id = reinterpret_cast<unsigned*>(after_stage);                   // [kDedupSlots]
  int* slot_pos = reinterpret_cast<int*>(slot_id + kDedupSlots);                   // [kDedupSlots]
  uint2* rep_addr = reinterpret_cast<uint2*>(slot_pos + kDedupSlots);              // [256]
  float* rep_score = reinterpret_cast<float*>(rep_addr + 256);                     // [256]
  int* slot_first = reinterpret_cast<int*>(rep_score + 256);                        // [kDedupSlots]
  int* wave_reps = slot_first + kDedupSlots;                                        // [4]
  if constexpr (DEDUP) {
    for (int i = threadIdx.x; i < kDedupSlots; i += 256) {
      slot_id[i] = kDedupEmpty;
      slot_first[i] = 0x7fffffff;
    }
  }

  stage_query<M>(lds, q1, q2, b, dim);  // (ends with a barrier: the tables are cleared)
  typename ModelOps<M>::Q q[NIT][VEC];
  load_query_regs<M, VEC, NIT, true>(lds, dim, ncol, lane, q);
  if constexpr (!DEDUP) {
    if (cnt <= 0) return;
  }
  int n_stream = cnt;        // rows this wavefront streams
  int first_rep = 0;         // DEDUP: position on the tile's list of the first of them
  int my_pos = lane;         // DEDUP: position on the list of the row my pair's score comes from
  if constexpr (DEDUP) {
    // The representative of an id is its first pair of the tile, and the list holds the representatives in pair
    // order: which wavefront scores which row is then the same in every run (a row's bits may depend on where it
    // stands in a wavefront's stream, through the contraction of multiply-adds in the unrolled row loop).
    const int pair_in_tile = wave * per_wave + lane;
    unsigned s = 0;
    if (lane < cnt) {
      const unsigned key = pb.row;
      s = (key * 2654435761u) >> 23;  // 9 bits
      while (true) {
        const unsigned old = atomicCAS(&slot_id[s], kDedupEmpty, key);
        if (old == kDedupEmpty || old == key) break;
        s = (s + 1) & (kDedupSlots - 1);
      }
      atomicMin(&slot_first[s], pair_in_tile);
    }
    __syncthreads();
    const bool is_rep = lane < cnt && slot_first[s] == pair_in_tile;
    const unsigned long long reps = __ballot(is_rep);
    if (lane == 0) wave_reps[wave] = __popcll(reps);
    __syncthreads();
    int before = 0, n_reps = 0;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const int c = wave_reps[w];
      before += w < wave ? c : 0;
      n_reps += c;
    }
    if (is_rep) {
      const int pos = before + (int)lanes_below_in(reps);
      slot_pos[s] = pos;
      const unsigned long long addr =
          (unsigned long long)(table + (((unsigned long long)pb.off_hi << 32) | pb.off_lo));
      rep_addr[pos] = make_uint2((unsigned)addr, (unsigned)(addr >> 32));
    }
    __syncthreads();
    if (lane < cnt) my_pos = slot_pos[s];
    const int share = (n_reps + 3) / 4;  // <= 64
    first_rep = wave * share;
    n_stream = max(0, min(share, n_reps - first_rep));
    // this wavefront's part of the list goes into its slab (entries past its end repeat the last: the row loop's
    // loads are unconditional)
    if (n_stream > 0) {
      *reinterpret_cast<uint2*>(slab + 4 * lane) = rep_addr[first_rep + min(lane, n_stream - 1)];
      slab_fence();
    }
  } else {
    stage_pairs(slab, lane, table, pb, 0.f, 0.f);
  }

  float neg_thr[NIT][VEC];
  if constexpr (CODED) {
#pragma unroll
    for (int it = 0; it < NIT; ++it)
#pragma unroll
      for (int v = 0; v < VEC; ++v) neg_thr[it][v] = ModelOps<M>::neg_threshold(q[it][v]);
  }
  float* out = score + (size_t)b * K + kw0;
  if (n_stream > 0)
  stream_batch<MUL, VEC, NIT, RIF>(slab, n_stream, dim, ncol, lane,
                                   [&](int j, const Pack<VEC>(&e1)[NIT], const Pack<VEC>(&e2)[NIT]) {
    // lanes past the row end hold a copy of the last column: they compute along and are dropped here.
    if constexpr (model_norm(M, REG)) {
      // unit-length halves: the two inner products and the two squared lengths are summed separately
      float dot1 = 0.f, dot2 = 0.f, sq1 = 0.f, sq2 = 0.f;
#pragma unroll
      for (int it = 0; it < NIT; ++it) {
        float a = 0.f, b2 = 0.f, c = 0.f, d = 0.f;
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
          a = __builtin_fmaf(e1[it].v[v], q[it][v].a, a);
          c = __builtin_fmaf(e1[it].v[v], e1[it].v[v], c);
          if constexpr (MUL == 2) {
            b2 = __builtin_fmaf(e2[it].v[v], q[it][v].b, b2);
            d = __builtin_fmaf(e2[it].v[v], e2[it].v[v], d);
          }
        }
        const bool in = lane + 64 * it < ncol;
        dot1 += in ? a : 0.f;
        dot2 += in ? b2 : 0.f;
        sq1 += in ? c : 0.f;
        sq2 += in ? d : 0.f;
      }
      dot1 = wave_sum_last_f32(dot1);
      sq1 = wave_sum_last_f32(sq1);
      float s = dot1 * inv_norm(sq1);
      if constexpr (MUL == 2) {
        dot2 = wave_sum_last_f32(dot2);
        sq2 = wave_sum_last_f32(sq2);
        s += dot2 * inv_norm(sq2);
      }
      s += p.gamma;
      if constexpr (DEDUP) {
        if (lane == 63) rep_score[first_rep + j] = s;
      } else {
        if (lane == 63) out[j] = s;
      }
      return;
    }
    // The logit is linear in the accumulators: fold them per lane, reduce once.
    float mine = 0.f;
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      float a0 = 0.f, a1 = 0.f;
      if constexpr (CODED) {
        unsigned code = 0;
#pragma unroll
        for (int v = 0; v < VEC; ++v) ModelOps<M>::fwd_coded(e1[it].v[v], q[it][v], neg_thr[it][v], a0, a1, code);
        stage[((DEDUP ? first_rep + j : j) & (kStaged - 1)) * (NIT * 64) + 64 * it + lane] = (unsigned char)code;
      } else {
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
          const float x1 = REG ? reg_apply(e1[it].v[v], p) : e1[it].v[v];
          const float x2 = MUL == 2 ? (REG ? reg_apply(e2[it].v[v], p) : e2[it].v[v]) : 0.f;
          ModelOps<M>::fwd(x1, x2, q[it][v], a0, a1);
        }
      }
      const float f = ModelOps<M>::fold(a0, a1, p);
      mine += lane + 64 * it < ncol ? f : 0.f;
    }
    const float folded = wave_sum_last_f32(mine);
    if constexpr (DEDUP) {
      if (lane == 63) rep_score[first_rep + j] = ModelOps<M>::score(folded, p);
    } else {
      if (lane == 63) out[j] = ModelOps<M>::score(folded, p);
      if constexpr (CODED) flush_codes<NIT>(stage, A.codes, (size_t)b * K + kw0, j, cnt, lane);
    }
  });
  if constexpr (DEDUP) {
    // every pair takes what its representative produced: the score from the tile's list ...
    __syncthreads();
    if (lane < cnt) out[lane] = rep_score[my_pos];
    if constexpr (CODED) {
      // ... and its NIT x 64 code bytes from the representative's row of the stage, 16 bytes per lane and turn;
      // the wavefront's pairs are contiguous in the code array
      if (cnt > 0) {
        typedef unsigned vec4u __attribute__((ext_vector_type(4)));
        constexpr int kPer = NIT * 4;  // 16-byte pieces per pair
        vec4u* dst = reinterpret_cast<vec4u*>(A.codes + ((size_t)b * K + kw0) * (size_t)(NIT * 64));
        for (int c0 = 0; c0 < cnt * kPer; c0 += 64) {
          const int c = c0 + lane;
          const int pair = min(c / kPer, cnt - 1);
          const int src_row = __shfl(my_pos, pair);
          if (c < cnt * kPer)
            __builtin_nontemporal_store(reinterpret_cast<const vec4u*>(stage + src_row * (NIT * 64))[c % kPer], dst + c);
        }
      }
    }
  }
  if (__ballot(bad != 0) != 0ull && err && lane == 0) *err = 1;
}

// SINGLES: the plan marks pairs whose entity occurs once in the step.  Such a segment needs no
// reduction, and this kernel already holds the pair's query in registers and has just read its entity
// row, so it finishes the row here (merged-gradient row and/or Adam on w, m, v) instead of leaving it
// to the entity pass, which would have to fetch the query rows and the entity row again.
// SINGLES: 0 = leave every segment to the entity pass, 1 = finish one-pair segments here as merged-gradient
// rows, 2 = ... with Adam on w, m, v (and the merged row if asked for).
// CODES (models with sign codes): 1 = also writes every pair's derivative decisions, one byte per lane
// and column group, for the entity pass to use in place of the query rows; 2 = the forward pass left
// the codes: the query gradient is summed from them and the entity rows are not read at all (except
// those of the one-pair segments finished here).
// GQ = false: only the one-pair segments are finished (optimizer on w, m, v); no query gradient, no
// other pair is touched.  The pairs' rows then come from the plan (uniq[segment]), not from the id tensor:
// this is the half of the work that smx_score_backward_entity hands to this kernel when the query
// gradients were taken earlier (autograd's backward) and the update comes later (apply_grad).
template <int M, int VEC, int NIT, int RIF, int NW, bool REG, int SINGLES, int CODES = 0, bool GQ = true>
__global__ __launch_bounds__(NW * 64) void score_backward_query_kernel(ScoreArgs A) {
  static_assert(GQ || (SINGLES == 2 && CODES == 0), "the one-pair-only form exists with an optimizer");
  const float* __restrict__ table = A.table;
  const long long* __restrict__ idx = A.idx;
  const float* __restrict__ q1 = A.q1;
  const float* __restrict__ q2 = A.q2;
  const float* __restrict__ score = A.score;
  const float* __restrict__ gscore = A.gscore;
  float* __restrict__ gq1 = A.gq1;
  float* __restrict__ gq2 = A.gq2;
  const int K = A.K, ncol = A.ncol;
  const unsigned long long n_rows = A.n_rows;
  const ScoreParams p = A.p;
  constexpr int MUL = model_mul(M);
  constexpr int NQ = model_nq(M);
  extern __shared__ float lds[];
  // Queries are taken last to first: the forward walks them first to last, and what it touched last -- the sign
  // codes it wrote, the rows it read -- is what the memory-side cache still holds when this kernel starts
  // (86 M x 200 box workload: backward 0.92 -> 0.91 ms; the kernel by itself, with nothing of a forward left in
  // that cache, takes 0.71 ms instead of 0.63).
  const int b = (int)(gridDim.x - 1u - blockIdx.x);
  const int lane = threadIdx.x & 63;
  const int wave = uniform(threadIdx.x >> 6);
  const int dim = ncol * VEC;
  const size_t row_len = (size_t)dim * MUL;

  stage_query<M>(lds, q1, q2, b, dim);
  typename ModelOps<M>::Q q[NIT][VEC];
  load_query_regs<M, VEC, NIT, false>(lds, dim, ncol, lane, q);

  float g1[NIT][VEC], g2[NIT][VEC];
  [[maybe_unused]] float neg_thr[NIT][VEC];  // sign-coded models, when this kernel makes the comparisons itself
#pragma unroll
  for (int it = 0; it < NIT; ++it)
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      g1[it][v] = g2[it][v] = 0.f;
      if constexpr (model_coded(M)) neg_thr[it][v] = ModelOps<M>::neg_threshold(q[it][v]);
    }
  // LDS: query | per-wavefront partial sums | per-wavefront pair slabs
  unsigned* slab = reinterpret_cast<unsigned*>(lds + (NW + 1) * NQ * dim) + wave * kSlabDwords;
  unsigned char* stage =
      reinterpret_cast<unsigned char*>(lds + (NW + 1) * NQ * dim + NW * kSlabDwords) + wave * (kStagePairs * NIT * 64);

  // this wavefront's share of the query's negatives: a contiguous range, walked in batches of 64
  const int per_wave = (K + NW - 1) / NW;
  const int kw0 = wave * per_wave;
  const int kw1 = min(K, kw0 + per_wave);
  int bad = 0;
  for (int kb = kw0; kb < kw1; kb += 64) {
    const int cnt = min(64, kw1 - kb);
    const size_t first = (size_t)(b / A.U) * K + kb;  // pairs belong to queries, a union's branch rows share them
    const size_t mine = first + min(lane, cnt - 1);
    int my_ps = 0;
    unsigned long long singles = 0ull;  // pairs of the batch that are a segment of their own
    if constexpr (SINGLES != 0) {
      my_ps = A.pair_seg[mine];
      singles = __ballot(lane < cnt && my_ps < 0);
    }
    PairBatch pb;
    if constexpr (GQ) {
      pb = load_pair_batch(idx, A.ids_shared ? (size_t)kb : first, cnt, lane, row_len, n_rows, bad);
    } else {
      if (singles == 0ull) continue;  // wave-uniform
      const unsigned long long row = my_ps < 0 ? (unsigned long long)A.uniq[my_ps & 0x7fffffff] : 0ull;
      const unsigned long long off = row * row_len;
      pb = PairBatch{(unsigned)off, (unsigned)(off >> 32), (unsigned)row};
    }
    float my_c0, my_c1;
    ModelOps<M>::coef(gscore[mine], score[mine], p, my_c0, my_c1);
    // Without optimizer state to fetch, such a pair's row is finished the moment it streams by: its entity
    // row and query are in registers, the merged-gradient row is one more store.
    constexpr bool kInStream = SINGLES == 1 && CODES != 2;
    // With the forward's codes and no optimizer the merged-gradient row of such a pair is a function of its
    // code bytes and coefficients alone: it is stored as the codes stream by, and the entity row is never read.
    constexpr bool kFromCodes = SINGLES == 1 && CODES == 2;
    if constexpr (!GQ) {
      // nothing streams: only the rows of the one-pair segments below
    } else if constexpr (CODES == 2) {
      // 8 pairs' code bytes requested at a time, two sets used in turn
      constexpr int CB = 8;
      const unsigned char* pc = A.codes_in + first * (size_t)(NIT * 64) + lane;
      unsigned ca[CB][NIT], cb[CB][NIT];
      auto request = [&](unsigned (&c)[CB][NIT], int j0) {
#pragma unroll
        for (int r = 0; r < CB; ++r) {
          const int j = min(j0 + r, cnt - 1);
#pragma unroll
          for (int it = 0; it < NIT; ++it) c[r][it] = pc[(size_t)j * (NIT * 64) + 64 * it];
        }
      };
      auto consume = [&](const unsigned (&c)[CB][NIT], int j0) {
#pragma unroll
        for (int r = 0; r < CB; ++r) {
          if (j0 + r < cnt) {
            const float c0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(my_c0), j0 + r));
            const float c1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(my_c1), j0 + r));
#pragma unroll
            for (int it = 0; it < NIT; ++it)
#pragma unroll
              for (int v = 0; v < VEC; ++v)
                ModelOps<M>::bwd_q_from_code(c0, c1, c[r][it], VEC - 1 - v, g1[it][v], g2[it][v]);
            if constexpr (kFromCodes) {
              if ((singles >> (j0 + r)) & 1ull) {  // wave-uniform
                RowRegs<MUL, VEC, NIT> none;
                float ge1[NIT][VEC], ge2[NIT][VEC];
#pragma unroll
                for (int it = 0; it < NIT; ++it)
#pragma unroll
                  for (int v = 0; v < VEC; ++v) {
                    none.h[0][it].v[v] = 0.f;
                    ge1[it][v] = ge2[it][v] = 0.f;
                    ModelOps<M>::bwd_e_coded(c0, c1, c[r][it], VEC - 1 - v, ge1[it][v]);
                  }
                const int seg = __builtin_amdgcn_readlane(my_ps, j0 + r) & 0x7fffffff;
                finish_row<M, VEC, NIT, REG, false>(A.sink, lane, 0u, seg, ge1, ge2, none, none, none);
              }
            }
          }
        }
      };
      request(ca, 0);
      for (int j0 = 0; j0 < cnt; j0 += 2 * CB) {
        request(cb, j0 + CB);
        consume(ca, j0);
        request(ca, j0 + 2 * CB);
        consume(cb, j0 + CB);
      }
    } else {
    stage_pairs(slab, lane, table, pb, my_c0, my_c1);
    int n_stream = cnt;
    if constexpr (SINGLES == 0 && CODES == 0) {
      if (A.winner) {  // uniform: a branch row of a union query streams the pairs it won, moved to the front of the slab
        const bool keep = lane < cnt && A.winner[mine] == (unsigned char)(b - (b / A.U) * A.U);
        const unsigned long long won = __ballot(keep);
        n_stream = __popcll(won);
        if (keep) {
          const unsigned long long addr =
              (unsigned long long)(table + (((unsigned long long)pb.off_hi << 32) | pb.off_lo));
          *reinterpret_cast<uint4*>(slab + 4 * lanes_below_in(won)) =
              make_uint4((unsigned)addr, (unsigned)(addr >> 32), __float_as_uint(my_c0), __float_as_uint(my_c1));
        }
        slab_fence();
      }
    }
    // lanes past the row end hold a copy of the last column: what they accumulate is never stored
    if (n_stream > 0)
    stream_batch<MUL, VEC, NIT, RIF>(slab, n_stream, dim, ncol, lane,
                                     [&](int j, const Pack<VEC>(&e1)[NIT], const Pack<VEC>(&e2)[NIT]) {
      float2 c = slab_coef(slab, j);
      [[maybe_unused]] const float c_raw = c.x;
      if constexpr (M == mL2)
        c.x = l2_pair_coef<VEC, NIT>(c.x, ncol, lane, [&](int it, int v) { return e1[it].v[v]; },
                                     [&](int it, int v) { return q[it][v].a; });
      if constexpr (model_norm(M, REG))  // d logit / d q = e / |e| per half: the upstream coefficient over the lengths
        c = norm_pair_coef<VEC, NIT, MUL>(c_raw, ncol, lane, [&](int it, int v) { return e1[it].v[v]; },
                                          [&](int it, int v) { return e2[it].v[v]; });
      if constexpr (CODES == 1) {
        // the pair's code bytes go to the wavefront's LDS stage, see flush_codes
        unsigned char* mine_b = stage + (j & (kStagePairs - 1)) * (NIT * 64) + lane;
#pragma unroll
        for (int it = 0; it < NIT; ++it) {
          unsigned code = 0;
#pragma unroll
          for (int v = 0; v < VEC; ++v)
            ModelOps<M>::bwd_q_coded(c.x, c.y, e1[it].v[v], q[it][v], neg_thr[it][v], g1[it][v], g2[it][v], code);
          mine_b[64 * it] = (unsigned char)code;
        }
        flush_codes<NIT>(stage, A.codes, first, j, cnt, lane);
      } else {
#pragma unroll
        for (int it = 0; it < NIT; ++it) {
#pragma unroll
          for (int v = 0; v < VEC; ++v) {
            const float x1 = REG ? reg_apply(e1[it].v[v], p) : e1[it].v[v];
            const float x2 = MUL == 2 ? (REG ? reg_apply(e2[it].v[v], p) : e2[it].v[v]) : 0.f;
            if constexpr (M == mBox) {
              ModelOps<M>::bwd_q_thr(c.x, c.y, x1, q[it][v], neg_thr[it][v], g1[it][v], g2[it][v]);
            } else if constexpr (model_norm(M, REG)) {
              g1[it][v] = __builtin_fmaf(c.x, x1, g1[it][v]);
              if constexpr (MUL == 2) g2[it][v] = __builtin_fmaf(c.y, x2, g2[it][v]);
            } else {
              ModelOps<M>::bwd_q(c.x, c.y, x1, x2, q[it][v], g1[it][v], g2[it][v]);
            }
          }
        }
      }
      if constexpr (kInStream) {
        if ((singles >> j) & 1ull) {  // wave-uniform
          RowRegs<MUL, VEC, NIT> w, none;
          float ge1[NIT][VEC], ge2[NIT][VEC];
#pragma unroll
          for (int it = 0; it < NIT; ++it)
#pragma unroll
            for (int v = 0; v < VEC; ++v) {
              w.h[0][it].v[v] = e1[it].v[v];
              if (MUL == 2) w.h[MUL - 1][it].v[v] = e2[it].v[v];
              ge1[it][v] = ge2[it][v] = 0.f;
              const float x1 = REG ? reg_apply(e1[it].v[v], p) : e1[it].v[v];
              const float x2 = MUL == 2 ? (REG ? reg_apply(e2[it].v[v], p) : e2[it].v[v]) : 0.f;
              ModelOps<M>::bwd_e(model_norm(M, REG) ? c_raw : c.x, c.y, x1, x2, q[it][v], ge1[it][v], ge2[it][v]);
            }
          const int seg = __builtin_amdgcn_readlane(my_ps, j) & 0x7fffffff;
          const unsigned row = (unsigned)__builtin_amdgcn_readlane((int)pb.row, j);
          finish_row<M, VEC, NIT, REG, false>(A.sink, lane, row, seg, ge1, ge2, w, none, none);
        }
      }
    });
    }

    if constexpr (SINGLES != 0 && !kInStream && !kFromCodes) {
      // S rows at a time per wavefront (their w, m, v loads are all requested before the first is
      // used): the row sets of the streaming loop are dead here, so this costs no extra registers, and
      // it divides the memory latency each one-pair row would otherwise expose by S.
      constexpr int S = NIT * MUL == 1 ? 3 : (NIT * MUL == 2 ? 2 : 1);
      unsigned long long todo = singles;
      while (todo != 0ull) {
        int js[S];
        RowRegs<MUL, VEC, NIT> e[S], m0[S], v0[S];
#pragma unroll
        for (int s = 0; s < S; ++s) {
          js[s] = todo != 0ull ? __builtin_ctzll(todo) : -1;
          if (js[s] >= 0) {  // wave-uniform
            todo &= todo - 1;
            const unsigned long long off = batch_off(pb, js[s]);
            load_row<MUL, VEC, NIT>(e[s], table + off, dim, ncol, lane);
            if constexpr (SINGLES == 2) {
              if (A.sink.adam_on == kOptAdam) load_row<MUL, VEC, NIT, true>(m0[s], A.sink.m + off, dim, ncol, lane);
              if (A.sink.adam_on != kOptSgd && !A.sink.squeeze)
                load_row<MUL, VEC, NIT, true>(v0[s], A.sink.v + off, dim, ncol, lane);
            }
          }
        }
#pragma unroll
        for (int s = 0; s < S; ++s) {
          if (js[s] >= 0) {
            const int j = js[s];
            float c0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(my_c0), j));
            const float c1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(my_c1), j));
            if constexpr (M == mL2)
              c0 = l2_pair_coef<VEC, NIT>(c0, ncol, lane, [&](int it, int v) { return e[s].h[0][it].v[v]; },
                                          [&](int it, int v) { return q[it][v].a; });
            const int seg = __builtin_amdgcn_readlane(my_ps, j) & 0x7fffffff;
            const unsigned row = (unsigned)__builtin_amdgcn_readlane((int)pb.row, j);
            float ge1[NIT][VEC], ge2[NIT][VEC];
#pragma unroll
            for (int it = 0; it < NIT; ++it)
#pragma unroll
              for (int v = 0; v < VEC; ++v) {
                ge1[it][v] = ge2[it][v] = 0.f;
                const float x1 = REG ? reg_apply(e[s].h[0][it].v[v], p) : e[s].h[0][it].v[v];
                const float x2 =
                    MUL == 2 ? (REG ? reg_apply(e[s].h[MUL - 1][it].v[v], p) : e[s].h[MUL - 1][it].v[v]) : 0.f;
                ModelOps<M>::bwd_e(c0, c1, x1, x2, q[it][v], ge1[it][v], ge2[it][v]);
              }
            finish_row<M, VEC, NIT, REG, SINGLES == 2>(A.sink, lane, row, seg, ge1, ge2, e[s], m0[s], v0[s]);
          }
        }
      }
    }
  }

  if constexpr (!GQ) return;
#pragma unroll
  for (int it = 0; it < NIT; ++it)
#pragma unroll
    for (int v = 0; v < VEC; ++v) finish_query_grad<M>(q[it][v], g1[it][v], g2[it][v], p);

  // wavefront partials -> LDS -> fixed-order sum over wavefronts
  float* part = lds + NQ * dim;  // [NW][NQ][dim]
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    const int c = lane + 64 * it;
    if (c < ncol) {
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        part[(wave * NQ + 0) * dim + c * VEC + v] = g1[it][v];
        if (NQ == 2) part[(wave * NQ + 1) * dim + c * VEC + v] = g2[it][v];
      }
    }
  }
  __syncthreads();
  for (int d = threadIdx.x; d < dim; d += NW * 64) {
    float s1 = 0.f, s2 = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      s1 += part[(w * NQ + 0) * dim + d];
      if (NQ == 2) s2 += part[(w * NQ + 1) * dim + d];
    }
    gq1[(size_t)b * dim + d] = s1;
    if (NQ == 2) gq2[(size_t)b * dim + d] = s2;
  }
}

// rows requested per batch; two batches are in flight at a time
constexpr int rows_in_flight(int nit, int mul) {
  const int r = 4 / (nit * mul);
  return r < 1 ? 1 : r;
}

template <int M, int VEC, int NIT, bool REG>
int launch_forward_reg(hipStream_t st, const ScoreArgs& A) {
  constexpr int RIF = rows_in_flight(NIT, model_mul(M));
  const size_t B = (size_t)A.B, K = (size_t)A.K;
  int tile_k = 256;  // 64 negatives per wavefront; smaller tiles when the grid would not fill the chip
  while (tile_k > 4 * RIF && (B * ((K + tile_k - 1) / tile_k) < 8192 || (size_t)tile_k / 2 >= K)) tile_k /= 2;
  const int tiles = (int)((K + tile_k - 1) / tile_k);
  const size_t lds = ((size_t)model_nq(M) * A.ncol * VEC + 4 * kSlabDwords) * sizeof(float);
  // ids given (not the dense layout, whose rows are all different): score each distinct entity of a
  // tile once
  // (not for a list of ids shared by the batch: a sampler's K negatives hardly ever repeat)
  const bool dedup = A.idx != nullptr && !A.ids_shared;
  if constexpr (model_coded(M) && !REG) {
    if (A.codes) {
      if (dedup)
        hipLaunchKernelGGL((score_forward_kernel<M, VEC, NIT, RIF, REG, true, true>), dim3((unsigned)(B * tiles)),
                           dim3(256), lds + 256 * NIT * 64 + kDedupLds, st, A, tiles, tile_k);
      else
        hipLaunchKernelGGL((score_forward_kernel<M, VEC, NIT, RIF, REG, true>), dim3((unsigned)(B * tiles)), dim3(256),
                           lds + 4 * kStagePairs * NIT * 64, st, A, tiles, tile_k);
      return check_launch("score forward (coded)");
    }
  }
  if (dedup)
    hipLaunchKernelGGL((score_forward_kernel<M, VEC, NIT, RIF, REG, false, true>), dim3((unsigned)(B * tiles)),
                       dim3(256), lds + kDedupLds, st, A, tiles, tile_k);
  else
    hipLaunchKernelGGL((score_forward_kernel<M, VEC, NIT, RIF, REG>), dim3((unsigned)(B * tiles)), dim3(256), lds, st, A,
                       tiles, tile_k);
  return check_launch("score forward");
}

template <int M, int VEC, int NIT, int NW, bool REG>
int launch_backward_query_reg(hipStream_t st, const ScoreArgs& A) {
  constexpr int RIF = rows_in_flight(NIT, model_mul(M));
  const size_t lds = ((size_t)(NW + 1) * model_nq(M) * A.ncol * VEC + NW * kSlabDwords) * sizeof(float);
  if (!A.gq1) {  // one-pair segments only; built for the shapes that have sign codes
    if constexpr (model_coded(M) && !REG && NW == 8 && NIT <= 2) {
      if (A.pair_seg && A.uniq && A.sink.adam_on) {
        hipLaunchKernelGGL((score_backward_query_kernel<M, VEC, NIT, RIF, NW, REG, 2, 0, false>), dim3((unsigned)A.B),
                           dim3(NW * 64), lds, st, A);
        return check_launch("score backward (one-pair segments)");
      }
    }
    return fail(SMX_ERR_ARG, "the one-pair-segment pass is not available for this model and shape");
  }
  if constexpr (model_coded(M) && !REG) {
    if (A.codes_in) {
      if (A.pair_seg && A.sink.adam_on)
        hipLaunchKernelGGL((score_backward_query_kernel<M, VEC, NIT, RIF, NW, REG, 2, 2>), dim3((unsigned)A.B),
                           dim3(NW * 64), lds, st, A);
      else if (A.pair_seg)
        hipLaunchKernelGGL((score_backward_query_kernel<M, VEC, NIT, RIF, NW, REG, 1, 2>), dim3((unsigned)A.B),
                           dim3(NW * 64), lds, st, A);
      else
        hipLaunchKernelGGL((score_backward_query_kernel<M, VEC, NIT, RIF, NW, REG, 0, 2>), dim3((unsigned)A.B),
                           dim3(NW * 64), lds, st, A);
      return check_launch("score backward (query, from codes)");
    }
    if (A.codes && A.pair_seg) {
      const size_t lds_coded = lds + (size_t)NW * kStagePairs * NIT * 64;
      if (A.sink.adam_on)
        hipLaunchKernelGGL((score_backward_query_kernel<M, VEC, NIT, RIF, NW, REG, 2, 1>), dim3((unsigned)A.B),
                           dim3(NW * 64), lds_coded, st, A);
      else
        hipLaunchKernelGGL((score_backward_query_kernel<M, VEC, NIT, RIF, NW, REG, 1, 1>), dim3((unsigned)A.B),
                           dim3(NW * 64), lds_coded, st, A);
      return check_launch("score backward (query, coded)");
    }
  }
  if (A.pair_seg && A.sink.adam_on)
    hipLaunchKernelGGL((score_backward_query_kernel<M, VEC, NIT, RIF, NW, REG, 2>), dim3((unsigned)A.B),
                       dim3(NW * 64), lds, st, A);
  else if (A.pair_seg)
    hipLaunchKernelGGL((score_backward_query_kernel<M, VEC, NIT, RIF, NW, REG, 1>), dim3((unsigned)A.B),
                       dim3(NW * 64), lds, st, A);
  else
    hipLaunchKernelGGL((score_backward_query_kernel<M, VEC, NIT, RIF, NW, REG, 0>), dim3((unsigned)A.B),
                       dim3(NW * 64), lds, st, A);
  return check_launch("score backward (query)");
}

template <int M, int VEC, int NIT>
int launch_score(hipStream_t st, const ScoreArgs& A, bool forward) {
  const bool reg = (M == mBetaKL && A.p.reg_on) || ((M == mComplex || M == mDistmult) && A.p.norm_on);
  if (forward) {
    if constexpr (M == mBetaKL || M == mComplex || M == mDistmult) {
      if (reg) return launch_forward_reg<M, VEC, NIT, true>(st, A);
    }
    return launch_forward_reg<M, VEC, NIT, false>(st, A);
  }
  // wavefronts per query: as many as 64 KiB of LDS allow -- the staged query and one partial-sum row per
  // wavefront, the wavefronts' 1 KiB pair slabs and, where the kernel writes sign codes, their code stages
  const size_t per_wave = (size_t)model_nq(M) * A.ncol * VEC * sizeof(float);
  const size_t extra = kSlabDwords * sizeof(unsigned) + (model_coded(M) ? (size_t)kStagePairs * NIT * 64 : 0);
  auto fits = [&](size_t n) { return (n + 1) * per_wave + n * extra <= 64 * 1024; };
  const int nw = fits(8) ? 8 : (fits(4) ? 4 : 2);
  if constexpr (M == mBetaKL || M == mComplex || M == mDistmult) {
    if (reg) {
      if (nw == 8) return launch_backward_query_reg<M, VEC, NIT, 8, true>(st, A);
      if (nw == 4) return launch_backward_query_reg<M, VEC, NIT, 4, true>(st, A);
      return launch_backward_query_reg<M, VEC, NIT, 2, true>(st, A);
    }
  }
  if (nw == 8) return launch_backward_query_reg<M, VEC, NIT, 8, false>(st, A);
  if (nw == 4) return launch_backward_query_reg<M, VEC, NIT, 4, false>(st, A);
  return launch_backward_query_reg<M, VEC, NIT, 2, false>(st, A);
}

// Instantiated once per model in its own translation unit (smx_score_inst_*.hip).
template <int M>
int score_dispatch(hipStream_t st, const ScoreArgs& A, int vec, int nit, bool forward) {
  if (vec == 4) {
    switch (nit) {
      case 1: return launch_score<M, 4, 1>(st, A, forward);
      case 2: return launch_score<M, 4, 2>(st, A, forward);
      case 4: return launch_score<M, 4, 4>(st, A, forward);
      default: return launch_score<M, 4, 8>(st, A, forward);
    }
  }
  switch (nit) {
    case 1: return launch_score<M, 1, 1>(st, A, forward);
    case 2: return launch_score<M, 1, 2>(st, A, forward);
    default: return launch_score<M, 1, 4>(st, A, forward);
  }
}

}  // namespace smx
