// Evaluation against all entities: filtered ranks of a query's answers without materialising or
// sorting the [1,N] logit row.
//
// Replaces, for the test_all case of smore/training/train_process.py:112-160,
//   negative_logit = model(None, all_entity_idx, ...)      score of every entity (kg_reasoning.py:349-355)
//   argsort(descending) -> ranking -> ranking[answers] -> sort -> minus arange -> +1   (filtered setting)
// The filtered rank of an answer is 1 + the number of NON-answer entities ranked before it.  So the
// table is streamed once, in order; a wavefront scores a row against the queries of the pass and
// finds, with one 64-bit compare per 64 answers, how many of the query's answers the entity does not
// beat; that number indexes a histogram (integer atomics: exact, order-free).  A prefix sum over the
// histogram gives every answer its count.  Order of equal scores: the lower entity id ranks first
// (one of the orders an unstable argsort may produce).  "Beats" is one unsigned compare of
// (sortable(score) << 32 | ~id) keys; the answers' keys come from the same scoring function.
#pragma once
#include "smx_common.h"
#include "smx_models.h"
#include "smx_wave.h"

namespace smx {

constexpr int kRankQueries = 4;  // most queries scored per pass over the table (short rows; 2 for long ones)

struct RankArgs {
  const float* table;
  const float* q1;
  const float* q2;
  int b0, B;            // queries [b0, b0 + NB) of B are handled by this launch (NB: see rank_scan_kernel)
  int U;                // union queries: q1 / q2 hold U branch rows per query, a logit is the maximum over them
                        // (the last line of every custom_cal_logit, smore/models/box.py:163); 1 otherwise
  int ncol;
  unsigned long long n_rows;
  ScoreParams p;
  // answers, per query A slots (the first ans_count[b] are valid), sorted by key descending for the scan
  const long long* ans_id;           // [B, A]
  const unsigned long long* ans_key; // [B, A]   (scan)
  unsigned long long* key_out;       // [B, A]   (answer-key kernel)
  float* score_out;                  // [B, A]   (answer-key kernel)
  const int* ans_count;              // [B]
  int A;
  unsigned* bins;                    // [B, A + 1]
  long long* rank_out;               // [B, A]
  // ranking among sampled candidates (rank_candidates_kernel)
  const long long* cand;             // [B, C], -1 = padding
  int C, H;
  const int* n_hard;                 // [B]: the first n_hard[b] candidates of query b are its hard answers
  float* cand_logit;                 // [B, C] or null
  long long* cand_rank;              // [B, C]
  long long* hard_rank;              // [B, H]
  int* err;
};

enum RankMode : int { kRankScan = 0, kRankKeys = 1, kRankCandidates = 2 };

__device__ __forceinline__ unsigned sortable_bits(float s) {
  const unsigned u = __float_as_uint(s);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);  // ascending in the float order (-0 < +0)
}
__device__ __forceinline__ unsigned long long rank_key(float score, unsigned long long id) {
  return ((unsigned long long)sortable_bits(score) << 32) | (unsigned)(~(unsigned)id);
}

// Whether branch logit s replaces the best so far: torch.max over the branch axis (a NaN wins, the first of equals stays).
__device__ __forceinline__ bool union_takes(float s, float best) { return s > best || (s != s && best == best); }

// Score of one row against one staged query; the value is valid in lane 63.
template <int M, int VEC, int NIT, bool REG>
__device__ __forceinline__ float row_score(const float (&e1)[NIT][VEC], const float (&e2)[NIT][VEC],
                                           const typename ModelOps<M>::Q (&q)[NIT][VEC], int ncol, int lane,
                                           const ScoreParams& p) {
  constexpr int MUL = model_mul(M);
  float mine = 0.f;
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    float a0 = 0.f, a1 = 0.f;
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      const float x1 = REG ? reg_apply(e1[it][v], p) : e1[it][v];
      const float x2 = MUL == 2 ? (REG ? reg_apply(e2[it][v], p) : e2[it][v]) : 0.f;
      ModelOps<M>::fwd(x1, x2, q[it][v], a0, a1);
    }
    const float f = ModelOps<M>::fold(a0, a1, p);
    mine += lane + 64 * it < ncol ? f : 0.f;
  }
  return ModelOps<M>::score(wave_sum_last_f32(mine), p);
}

// ComplEx with unit-length halves (REG stands for it there): the row's halves scaled in the lanes' registers, once
// per row however many queries score it.
template <int M, int VEC, int NIT, bool REG>
__device__ __forceinline__ void unit_row(float (&e1)[NIT][VEC], float (&e2)[NIT][VEC], int ncol, int lane) {
  if constexpr (model_norm(M, REG)) {
    float s1 = 0.f, s2 = 0.f;
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      float a = 0.f, b = 0.f;
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        a = __builtin_fmaf(e1[it][v], e1[it][v], a);
        if constexpr (model_mul(M) == 2) b = __builtin_fmaf(e2[it][v], e2[it][v], b);
      }
      const bool in = lane + 64 * it < ncol;
      s1 += in ? a : 0.f;
      s2 += in ? b : 0.f;
    }
    const float i1 = inv_norm(wave_sum_f32(s1));
    const float i2 = model_mul(M) == 2 ? inv_norm(wave_sum_f32(s2)) : 0.f;
#pragma unroll
    for (int it = 0; it < NIT; ++it)
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        e1[it][v] *= i1;
        if constexpr (model_mul(M) == 2) e2[it][v] *= i2;
      }
  }
}

// STREAM: the row is read once in a pass over the whole table (non-temporal load).
template <int VEC, int NIT, int MUL, bool STREAM = false>
__device__ __forceinline__ void load_entity(const float* __restrict__ row, int dim, int ncol, int lane,
                                            float (&e1)[NIT][VEC], float (&e2)[NIT][VEC]) {
  typedef float vec4f __attribute__((ext_vector_type(4)));
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    const int c = min(lane + 64 * it, ncol - 1);
    if constexpr (VEC == 4) {
      const vec4f* pa = reinterpret_cast<const vec4f*>(row) + c;
      const vec4f a = STREAM ? __builtin_nontemporal_load(pa) : *pa;
      e1[it][0] = a.x; e1[it][1] = a.y; e1[it][2] = a.z; e1[it][3] = a.w;
      if (MUL == 2) {
        const vec4f* pb = reinterpret_cast<const vec4f*>(row + dim) + c;
        const vec4f b = STREAM ? __builtin_nontemporal_load(pb) : *pb;
        e2[it][0] = b.x; e2[it][1] = b.y; e2[it][2] = b.z; e2[it][3] = b.w;
      }
    } else {
      e1[it][0] = STREAM ? __builtin_nontemporal_load(row + c) : row[c];
      if (MUL == 2) e2[it][0] = STREAM ? __builtin_nontemporal_load(row + dim + c) : row[dim + c];
    }
  }
}

template <int M, int VEC, int NIT>
__device__ __forceinline__ void load_rank_query(const float* __restrict__ q1, const float* __restrict__ q2, int b,
                                                int dim, int ncol, int lane,
                                                typename ModelOps<M>::Q (&q)[NIT][VEC]) {
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    const int c = min(lane + 64 * it, ncol - 1);
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      const float a = q1[(size_t)b * dim + c * VEC + v];
      const float bb = model_nq(M) == 2 ? q2[(size_t)b * dim + c * VEC + v] : 0.f;
      q[it][v] = prep_forward<M>(a, bb);
    }
  }
}

// Keys (and scores) of the answers: one wavefront per (query, answer slot).
template <int M, int VEC, int NIT, bool REG>
__global__ __launch_bounds__(256) void rank_answer_keys_kernel(RankArgs A) {
  constexpr int MUL = model_mul(M);
  const int lane = threadIdx.x & 63;
  const int slot = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (slot >= A.B * A.A) return;
  const int b = slot / A.A, j = slot - b * A.A;
  const int dim = A.ncol * VEC;
  const bool valid = j < A.ans_count[b];
  unsigned long long id = valid ? (unsigned long long)A.ans_id[slot] : 0ull;
  if (id >= A.n_rows) id = 0;  // the host wrapper has already refused such ids
  typename ModelOps<M>::Q q[NIT][VEC];
  float e1[NIT][VEC], e2[NIT][VEC];
  load_entity<VEC, NIT, MUL>(A.table + id * (size_t)dim * MUL, dim, A.ncol, lane, e1, e2);
  unit_row<M, VEC, NIT, REG>(e1, e2, A.ncol, lane);
  float s = 0.f;
  for (int u = 0; u < A.U; ++u) {  // uniform
    load_rank_query<M, VEC, NIT>(A.q1, A.q2, b * A.U + u, dim, A.ncol, lane, q);
    const float su = row_score<M, VEC, NIT, REG>(e1, e2, q, A.ncol, lane, A.p);
    if (u == 0 || union_takes(su, s)) s = su;
  }
  if (lane == 63) {
    A.score_out[slot] = valid ? s : 0.f;
    A.key_out[slot] = valid ? rank_key(s, id) : 0ull;  // key 0 sorts last and is never counted
  }
}

// The scan for NB (1, 2 or 4) queries -- or, UNION, for ONE query whose NB register sets hold its branch rows (a
// set past the last branch repeats it): an entity's logit is then the maximum over the sets, and there is one list
// of answers.  LDS: bins [NL][A + 1], keys [NL][A] with NL = the number of answer lists (NB, or 1).
template <int M, int VEC, int NIT, bool REG, int NB, bool UNION = false>
__global__ __launch_bounds__(256) void rank_scan_kernel(RankArgs A) {
  constexpr int NL = UNION ? 1 : NB;
  constexpr int MUL = model_mul(M);
  constexpr int RIF = NIT * MUL <= 2 ? 4 : (NIT * MUL <= 4 ? 2 : 1);
  extern __shared__ unsigned lds_bins[];  // bins [NB][A + 1], then (8-byte aligned) the answers' keys [NB][A]
  const int lane = threadIdx.x & 63;
  const int wave = uniform(threadIdx.x >> 6);
  const int dim = A.ncol * VEC;
  const size_t row_len = (size_t)dim * MUL;
  const int A1 = A.A + 1;
  unsigned long long* lds_keys = reinterpret_cast<unsigned long long*>(lds_bins + ((NL * A1 + 1) & ~1));
  for (int i = threadIdx.x; i < NL * A1; i += 256) lds_bins[i] = 0u;
  for (int i = threadIdx.x; i < NL * A.A; i += 256) {
    const int x = i / A.A, j = i - x * A.A;
    const int b = min(A.b0 + x, A.B - 1);
    lds_keys[i] = j < A.ans_count[b] ? A.ans_key[(size_t)b * A.A + j] : 0ull;
  }
  __syncthreads();

  typename ModelOps<M>::Q q[NB][NIT][VEC];
  int count[NL], qb[NL];
#pragma unroll
  for (int x = 0; x < NL; ++x) {
    qb[x] = min(A.b0 + x, A.B - 1);  // a pass past the last query repeats it; its histogram is dropped
    count[x] = min(max(A.ans_count[qb[x]], 0), A.A);  // a count beyond the slots would index past the LDS arrays
  }
#pragma unroll
  for (int x = 0; x < NB; ++x)
    load_rank_query<M, VEC, NIT>(A.q1, A.q2, UNION ? qb[0] * A.U + min(x, A.U - 1) : qb[x], dim, A.ncol, lane, q[x]);
  const int chunks = (A.A + 63) / 64;
  // The first 64 answers' keys stay in registers (most queries have no more); further chunks come from LDS.
  // live[x]: lanes that hold one of them.  my_id[x]: that answer's entity id.
  unsigned long long first_keys[NL], live[NL];
  unsigned my_id[NL];
  // tally[x], lane L: rows so far that beat exactly L of query x's answers (the common cases: L = 0 is
  // every entity ranked below all answers).  Rows that beat 64 or more go to the LDS histogram directly.
  unsigned tally[NL];
#pragma unroll
  for (int x = 0; x < NL; ++x) {
    first_keys[x] = lane < count[x] ? lds_keys[x * A.A + lane] : 0ull;
    live[x] = count[x] >= 64 ? ~0ull : ((1ull << count[x]) - 1ull);
    my_id[x] = (unsigned)~(unsigned)first_keys[x];
    tally[x] = 0u;
  }

  // Wavefronts walk the table together: group g of RIF consecutive rows belongs to wavefront g mod n_waves.
  // Group and row numbers are 32-bit scalars (the host refuses tables of 2^32 - 8 rows or more).  Requests
  // are unconditional -- past the end they repeat the last group -- and rows past the end are scored and
  // then dropped, so that no branch separates a request from the use of the rows requested before it:
  // the counters the compiler waits on then leave the newest RIF loads in flight.
  const unsigned n_waves = gridDim.x * 4u;
  const unsigned wid = blockIdx.x * 4u + (unsigned)wave;
  const unsigned n_rows32 = (unsigned)A.n_rows;
  const unsigned groups = (n_rows32 + RIF - 1) / RIF;
  float ea1[RIF][NIT][VEC], ea2[RIF][NIT][VEC], eb1[RIF][NIT][VEC], eb2[RIF][NIT][VEC];
  auto request = [&](float (&x1)[RIF][NIT][VEC], float (&x2)[RIF][NIT][VEC], unsigned g) {
    g = min(g, groups - 1);
#pragma unroll
    for (int r = 0; r < RIF; ++r) {
      const unsigned row = min(g * RIF + r, n_rows32 - 1);
      load_entity<VEC, NIT, MUL, true>(A.table + row * row_len, dim, A.ncol, lane, x1[r], x2[r]);
    }
  };
  auto consume = [&](const float (&x1)[RIF][NIT][VEC], const float (&x2)[RIF][NIT][VEC], unsigned g) {
#pragma unroll
    for (int r = 0; r < RIF; ++r) {
      const unsigned id = g * RIF + r;  // entity id of the row
      float u1[NIT][VEC], u2[NIT][VEC];  // (the row itself unless the model scales it)
#pragma unroll
      for (int it = 0; it < NIT; ++it)
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
          u1[it][v] = x1[r][it][v];
          u2[it][v] = MUL == 2 ? x2[r][it][v] : 0.f;
        }
      unit_row<M, VEC, NIT, REG>(u1, u2, A.ncol, lane);
#pragma unroll
      for (int x = 0; x < NL; ++x) {
        const float s = row_score<M, VEC, NIT, REG>(u1, u2, q[x], A.ncol, lane, A.p);
        float su = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(s), 63));
        if constexpr (UNION) {
#pragma unroll
          for (int u = 1; u < NB; ++u) {
            const float t = row_score<M, VEC, NIT, REG>(u1, u2, q[u], A.ncol, lane, A.p);
            const float tu = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(t), 63));
            if (union_takes(tu, su)) su = tu;
          }
        }
        const unsigned long long key = rank_key(su, id);
        int not_beaten = __popcll(__ballot(!(key > first_keys[x])) & live[x]);
        bool skip = id >= n_rows32 || (__ballot(my_id[x] == id) & live[x]) != 0ull;  // past the end, or an answer
        for (int c = 1; c < chunks; ++c) {
          const int j = c * 64 + lane;
          const bool in_list = j < count[x];
          const unsigned long long ak = in_list ? lds_keys[x * A.A + j] : 0ull;
          not_beaten += __popcll(__ballot(in_list && !(key > ak)));
          skip |= __ballot(in_list && ((unsigned)~(unsigned)ak == id)) != 0ull;
        }
        const int beaten = skip ? -1 : count[x] - not_beaten;  // wave-uniform; -1 matches no lane
        tally[x] += lane == beaten ? 1u : 0u;
        if (beaten >= 64 && lane == 0) atomicAdd(&lds_bins[x * A1 + not_beaten], 1u);
      }
    }
  };
  if (wid < groups) {
    unsigned g = wid;
    request(ea1, ea2, g);
    while (true) {
      // (group numbers stay below 2^30 + 2 * n_waves: no wrap-around)
      request(eb1, eb2, g + n_waves);
      consume(ea1, ea2, g);
      if (g + n_waves >= groups) break;
      request(ea1, ea2, g + 2 * n_waves);
      consume(eb1, eb2, g + n_waves);
      if (g + 2 * n_waves >= groups) break;
      g += 2 * n_waves;
    }
  }
#pragma unroll
  for (int x = 0; x < NL; ++x)
    if (lane <= count[x] && tally[x] != 0u) atomicAdd(&lds_bins[x * A1 + (count[x] - lane)], tally[x]);
  __syncthreads();
#pragma unroll
  for (int x = 0; x < NL; ++x) {
    if (A.b0 + x < A.B) {
      for (int i = threadIdx.x; i < A1; i += 256) {
        const unsigned v = lds_bins[x * A1 + i];
        if (v) atomicAdd(&A.bins[(size_t)(A.b0 + x) * A1 + i], v);
      }
    }
  }
}

// Evaluation against sampled candidates (the branch of smore/training/train_process.py:118-128 taken when the
// evaluation set brings its own negatives): one workgroup per query scores the query's C candidates -- padding
// (-1) is scored as entity 0 with a bias of -1e6 added to the logit, exactly as the reference does -- and ranks
// them among themselves: ranking[j] = number of candidates ordered before candidate j by descending biased
// logit, i.e. the position `argsort(descending)` gives it (equal logits: the lower position first, one of the
// orders an unstable argsort may produce).  The first n_hard candidates are the hard answers; their filtered
// ranks (rank - number of hard answers ranked before it + 1, :141-145) come out as well.
// LDS: keys [C] (64-bit), ranks of the hard answers [H].
constexpr int kCandThreads = 1024;

template <int M, int VEC, int NIT, bool REG>
__global__ __launch_bounds__(kCandThreads) void rank_candidates_kernel(RankArgs A) {
  constexpr int MUL = model_mul(M);
  extern __shared__ unsigned long long cand_keys[];  // [C], then int ranks [H]
  int* hard_ranks = reinterpret_cast<int*>(cand_keys + A.C);
  const int b = blockIdx.x;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int dim = A.ncol * VEC;
  typename ModelOps<M>::Q q[NIT][VEC];
  load_rank_query<M, VEC, NIT>(A.q1, A.q2, b * A.U, dim, A.ncol, lane, q);  // (the first branch, or the only one)
  int bad = 0;
  for (int j = wave; j < A.C; j += kCandThreads / 64) {  // uniform per wavefront
    const long long raw = A.cand[(size_t)b * A.C + j];
    const bool pad = raw == -1;
    unsigned long long id = pad ? 0ull : (unsigned long long)raw;
    if (id >= A.n_rows) {
      bad = 1;
      id = 0;
    }
    float e1[NIT][VEC], e2[NIT][VEC];
    load_entity<VEC, NIT, MUL>(A.table + id * (size_t)dim * MUL, dim, A.ncol, lane, e1, e2);
    unit_row<M, VEC, NIT, REG>(e1, e2, A.ncol, lane);
    float s = row_score<M, VEC, NIT, REG>(e1, e2, q, A.ncol, lane, A.p);
    for (int u = 1; u < A.U; ++u) {  // uniform: the other branches of a union query, fetched again per candidate
      typename ModelOps<M>::Q qu[NIT][VEC];
      load_rank_query<M, VEC, NIT>(A.q1, A.q2, b * A.U + u, dim, A.ncol, lane, qu);
      const float su = row_score<M, VEC, NIT, REG>(e1, e2, qu, A.ncol, lane, A.p);
      if (union_takes(su, s)) s = su;
    }
    s += pad ? -1e6f : 0.f;
    if (lane == 63) {
      if (A.cand_logit) A.cand_logit[(size_t)b * A.C + j] = s;
      cand_keys[j] = ((unsigned long long)sortable_bits(s) << 32) | (unsigned)(~(unsigned)j);
    }
  }
  if (bad && A.err && lane == 0) *A.err = 1;
  __syncthreads();
  const int n_hard = min(A.n_hard[b], min(A.H, A.C));
  for (int j = threadIdx.x; j < A.C; j += kCandThreads) {
    const unsigned long long mine = cand_keys[j];
    int before = 0;
    for (int i = 0; i < A.C; ++i) before += cand_keys[i] > mine ? 1 : 0;  // every thread reads the same key: a broadcast
    A.cand_rank[(size_t)b * A.C + j] = before;
    if (j < n_hard) hard_ranks[j] = before;
  }
  __syncthreads();
  for (int j = threadIdx.x; j < A.H; j += kCandThreads) {
    long long out = 0;
    if (j < n_hard) {
      const int mine = hard_ranks[j];
      int ahead = 0;
      for (int i = 0; i < n_hard; ++i) ahead += hard_ranks[i] < mine ? 1 : 0;
      out = (long long)(mine - ahead + 1);
    }
    A.hard_rank[(size_t)b * A.H + j] = out;
  }
}

static __global__ __launch_bounds__(256) void rank_clear_kernel(unsigned* bins, size_t n) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) bins[i] = 0u;
}

// filtered rank of answer j (in key order) = 1 + sum of the bins 0..j; one workgroup per query
static __global__ __launch_bounds__(256) void rank_finish_kernel(RankArgs A) {
  const int b = blockIdx.x;
  const int A1 = A.A + 1;
  if (threadIdx.x == 0) {
    unsigned long long run = 0;
    const int n = A.ans_count[b];
    for (int j = 0; j < A.A; ++j) {
      run += A.bins[(size_t)b * A1 + j];
      A.rank_out[(size_t)b * A.A + j] = j < n ? (long long)(run + 1ull) : 0ll;
    }
  }
}

template <int M, int VEC, int NIT, bool REG>
int launch_rank_reg(hipStream_t st, RankArgs A, int mode) {
  if (mode == kRankCandidates) {
    const size_t lds = (size_t)A.C * sizeof(unsigned long long) + (size_t)A.H * sizeof(int);
    hipLaunchKernelGGL((rank_candidates_kernel<M, VEC, NIT, REG>), dim3((unsigned)A.B), dim3(kCandThreads), lds, st, A);
    return check_launch("rank candidates");
  }
  if (mode == kRankKeys) {
    const unsigned blocks = (unsigned)(((size_t)A.B * A.A + 3) / 4);
    hipLaunchKernelGGL((rank_answer_keys_kernel<M, VEC, NIT, REG>), dim3(blocks), dim3(256), 0, st, A);
    return check_launch("rank answer keys");
  }
  const size_t n_bins = (size_t)A.B * (A.A + 1);
  hipLaunchKernelGGL(rank_clear_kernel, dim3((unsigned)((n_bins + 255) / 256)), dim3(256), 0, st, A.bins, n_bins);
  int dev = 0, cus = 256;
  if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  auto lds_bytes = [&](int nb) {
    return (((size_t)nb * (A.A + 1) + 1) & ~(size_t)1) * sizeof(unsigned) + (size_t)nb * A.A * sizeof(unsigned long long);
  };
  auto grid_for = [&](auto kernel, size_t lds) {
    int per_cu = 2;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, 256, lds) != hipSuccess || per_cu < 1) per_cu = 2;
    unsigned blocks = (unsigned)cus * (unsigned)per_cu;
    const unsigned long long want = (A.n_rows + 15) / 16;
    if (want < blocks) blocks = (unsigned)(want ? want : 1);
    return blocks;
  };
  // Queries per pass: the row is fetched once for all of them, and the kernel turns from bandwidth-bound
  // to issue-bound between one and two.  Four when the rows are short enough for four queries' registers
  // and the answers' keys and histograms of four queries fit 48 KB of LDS.
  constexpr bool kFourFit = NIT * model_mul(M) <= 2;
  if (A.U > 1) {  // union queries: one query per pass, its branch rows in the register sets
    if (A.U > 2 && !kFourFit)
      return fail(SMX_ERR_SHAPE, "union queries of %d branches over rows this long are not supported by the scan (2 at most)", A.U);
    for (int b0 = 0; b0 < A.B; ++b0) {
      A.b0 = b0;
      const size_t lds = lds_bytes(1);
      if (A.U == 2) {
        hipLaunchKernelGGL((rank_scan_kernel<M, VEC, NIT, REG, 2, true>),
                           dim3(grid_for(rank_scan_kernel<M, VEC, NIT, REG, 2, true>, lds)), dim3(256), lds, st, A);
      } else if constexpr (kFourFit) {
        hipLaunchKernelGGL((rank_scan_kernel<M, VEC, NIT, REG, 4, true>),
                           dim3(grid_for(rank_scan_kernel<M, VEC, NIT, REG, 4, true>, lds)), dim3(256), lds, st, A);
      }
    }
    hipLaunchKernelGGL(rank_finish_kernel, dim3((unsigned)A.B), dim3(256), 0, st, A);
    return check_launch("rank scan (union queries)");
  }
  for (int b0 = 0; b0 < A.B;) {
    A.b0 = b0;
    const int left = A.B - b0;
    if (kFourFit && left >= 4 && lds_bytes(4) <= (size_t)48 << 10) {
      if constexpr (kFourFit) {
        const size_t lds = lds_bytes(4);
        hipLaunchKernelGGL((rank_scan_kernel<M, VEC, NIT, REG, 4>),
                           dim3(grid_for(rank_scan_kernel<M, VEC, NIT, REG, 4>, lds)), dim3(256), lds, st, A);
      }
      b0 += 4;
    } else if (left >= 2) {
      const size_t lds = lds_bytes(2);
      hipLaunchKernelGGL((rank_scan_kernel<M, VEC, NIT, REG, 2>), dim3(grid_for(rank_scan_kernel<M, VEC, NIT, REG, 2>, lds)),
                         dim3(256), lds, st, A);
      b0 += 2;
    } else {
      const size_t lds = lds_bytes(1);
      hipLaunchKernelGGL((rank_scan_kernel<M, VEC, NIT, REG, 1>), dim3(grid_for(rank_scan_kernel<M, VEC, NIT, REG, 1>, lds)),
                         dim3(256), lds, st, A);
      b0 += 1;
    }
  }
  hipLaunchKernelGGL(rank_finish_kernel, dim3((unsigned)A.B), dim3(256), 0, st, A);
  return check_launch("rank scan");
}

template <int M, int VEC, int NIT>
int launch_rank(hipStream_t st, const RankArgs& A, int mode) {
  if constexpr (M == mBetaKL || M == mComplex || M == mDistmult) {
    if (M == mBetaKL ? A.p.reg_on : A.p.norm_on) return launch_rank_reg<M, VEC, NIT, true>(st, A, mode);
  }
  return launch_rank_reg<M, VEC, NIT, false>(st, A, mode);
}

// Instantiated once per model in its own translation unit (smx_rank_inst_*.hip).
template <int M>
int rank_dispatch(hipStream_t st, const RankArgs& A, int vec, int nit, int mode) {
  if (vec == 4) {
    switch (nit) {
      case 1: return launch_rank<M, 4, 1>(st, A, mode);
      case 2: return launch_rank<M, 4, 2>(st, A, mode);
      case 4: return launch_rank<M, 4, 4>(st, A, mode);
      default: return launch_rank<M, 4, 8>(st, A, mode);
    }
  }
  switch (nit) {
    case 1: return launch_rank<M, 1, 1>(st, A, mode);
    case 2: return launch_rank<M, 1, 2>(st, A, mode);
    default: return launch_rank<M, 1, 4>(st, A, mode);
  }
}

}  // namespace smx
