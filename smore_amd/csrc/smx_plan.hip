// Segment plan: groups the (query, negative) pairs of one step by entity id.
//
// Replaces merge_grad_indices (smore/common/embedding/embed_optimizer.py:39-42),
// i.e. torch.unique(ids, return_inverse=True), which the reference runs on the
// host CPU, with a device pipeline of six kernel launches and nothing else (no
// library sort, no memset: the whole build can be recorded into a HIP graph):
//   hist    one read of the ids: range check, digit histograms of every radix pass per tile of the passes,
//           zero fill of the tables the later kernels count in
//   sum     digit counts of every pass over the whole input; for the first pass also per tile the
//           counts of the tiles before it
//   pass    x (key bits / digit bits): stable LSD radix pass over (id, pair) as one 64-bit element
//   emit    segment heads, segment numbers, uniq, seg_start, inverse, pair_seg, n_uniq
// The sort is written for this shape: keys are entity ids (only the bits an id below n_rows can
// have are sorted, 27 for 86M rows = three 9-bit passes), the payload is the pair index and is
// also the tie-break, so inside a segment pairs stay in ascending pair order and every later
// reduction over a segment has one fixed summation order.
//
// A radix pass handles a tile of up to 18432 elements per workgroup of 1024 threads: elements are
// kept in registers, ranked per wavefront with ballot matching (stable: lane order inside a round,
// rounds in order, wavefronts in order), the tile is reordered in LDS and written out in digit runs.
// Where a digit's run starts in the output depends on the tiles before: the first pass reads that from
// the sum kernel's table; in the later passes a tile publishes its digit counts and reads back the counts
// of the tiles before it ("look-back"; tiles take their number from a ticket counter, so a tile only ever
// waits for tiles that are already running).  Waiting is bounded: a tile that would wait too long gives
// up, marks the plan invalid (*err_flag = 2, n_uniq = -1) and every kernel still ends.
//
// An id outside [0, n_rows) sets *err_flag = 1 and gets the key n_rows: such pairs sort behind
// every valid id, form a last segment of their own that is not counted in n_uniq and that the
// entity pass skips, and are never marked as one-pair segments -- no table row is updated for them.
#include <cstring>
#include <mutex>

#include "../../include/smx_measure.h"
#include "smx_common.h"

namespace smx {

constexpr int kSortMaxRounds = 18;          // elements per thread and tile
constexpr int kSortMaxDigitBits = 10;
constexpr int kGroup = 16;                  // look-back fan-in: tiles per group, groups per super-block, ...
constexpr unsigned kReady = 0x80000000u;    // published words: flag | 31-bit count
constexpr unsigned kCount = 0x7fffffffu;
constexpr unsigned kSpinLimit = 1u << 22;   // polls before a waiting tile gives up
constexpr int kAuxThreads = 1024;           // workgroup size of the hist, sum and emit kernels
constexpr int kAuxWaves = kAuxThreads / 64;
constexpr int kHistBatch = 6;               // ids a thread of the hist kernel requests at a time
constexpr int kEmitIters = 16;              // sorted positions per thread of the emit kernel, at most (see emit_iters)
constexpr int kEmitSuper = 256;             // emit tiles whose head counts one wavefront reads back at once

__device__ __forceinline__ unsigned ld_agent(const unsigned* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_agent(unsigned* p, unsigned v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Waits until the word at p carries the ready flag; v is what was last read there.  Bounded: after
// spin_limit polls the caller gets a ready word with count 0, gave_up is set and the plan is marked invalid.
__device__ __forceinline__ unsigned wait_ready(const unsigned* p, unsigned v, unsigned* abort_flag, int* err,
                                               unsigned spin_limit, unsigned& gave_up) {
  unsigned spins = 0;
  while (!(v & kReady)) {
    __builtin_amdgcn_s_sleep(1);
    v = ld_agent(p);
    if (++spins > spin_limit) {
      st_agent(abort_flag, 1u);
      if (err) *err = 2;
      gave_up = 1u;
      return kReady;
    }
  }
  return v;
}

// Orders a wavefront's own LDS writes before its later LDS reads (other lanes' entries).
__device__ __forceinline__ void wave_lds_fence() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Exclusive prefix, in thread order, of one value per thread of a workgroup of NW wavefronts; *total
// (may be null) gets the sum.  tmp: NW words of LDS.
template <int NW>
__device__ __forceinline__ unsigned block_excl_scan(unsigned v, unsigned* tmp, unsigned* total) {
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  unsigned inc = v;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const unsigned t = __shfl_up(inc, off);
    if (lane >= off) inc += t;
  }
  __syncthreads();  // tmp may still be read from an earlier scan
  if (lane == 63) tmp[w] = inc;
  __syncthreads();
  unsigned before = 0, all = 0;
#pragma unroll
  for (int i = 0; i < NW; ++i) {
    const unsigned t = tmp[i];
    before += i < w ? t : 0u;
    all += t;
  }
  if (total) *total = all;
  return before + inc - v;
}

__device__ __forceinline__ unsigned clamp_id(long long id, unsigned long long n_rows, int& bad) {
  if ((unsigned long long)id >= n_rows) {
    bad = 1;
    return (unsigned)n_rows;
  }
  return (unsigned)id;
}

// Lanes of the wavefront (among those of `live`) whose `bits`-bit digit equals this lane's: one ballot
// per bit, combined with a three-input bit operation per half (same & ~(has ^ mine)).
__device__ __forceinline__ unsigned long long match_digit(unsigned d, int bits, unsigned long long live) {
  unsigned lo = (unsigned)live, hi = (unsigned)(live >> 32);
#pragma unroll
  for (int b = 0; b < kSortMaxDigitBits; ++b) {
    if (b < bits) {  // uniform
      const unsigned mine = (unsigned)__builtin_amdgcn_sbfe((int)d, b, 1);  // 0 or ~0
      const unsigned long long has = __ballot(mine != 0u);
      lo = __builtin_amdgcn_bitop3_b32(lo, (unsigned)has, mine, 0x90);
      hi = __builtin_amdgcn_bitop3_b32(hi, (unsigned)(has >> 32), mine, 0x90);
    }
  }
  return ((unsigned long long)hi << 32) | lo;
}
__device__ __forceinline__ unsigned lanes_below(unsigned long long m) {
  return __builtin_amdgcn_mbcnt_hi((unsigned)(m >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)m, 0u));
}

// ---- hist -------------------------------------------------------------------------------------
// block_hist[tile][pass][digit]: how many ids of a tile of the radix passes (tile_len consecutive ids, one
// workgroup each) have that digit in that pass.  The first pass takes its tiles' counts from here and needs no
// look-back; the later passes need the counts of the whole input only (their tiles hold other elements).
// Ids are skewed (a few entities collect most pairs, and the high digits of small ids are all zero):
// lanes that share the first lane's digit are counted with one LDS atomic for all of them.
__device__ __forceinline__ void count_digit(unsigned* hist, unsigned d, bool valid, int lane) {
  const unsigned long long live = __ballot(valid);
  if (live == 0ull) return;  // uniform
  const unsigned d0 = (unsigned)__builtin_amdgcn_readlane((int)d, __builtin_ctzll(live));
  const unsigned long long like_first = __ballot(valid && d == d0);
  if (valid) {
    if (d != d0) atomicAdd(&hist[d], 1u);
    else if (lane == __builtin_ctzll(like_first)) atomicAdd(&hist[d], (unsigned)__popcll(like_first));
  }
}

__global__ __launch_bounds__(kAuxThreads) void sort_hist_kernel(const long long* __restrict__ idx, int n, int tile_len,
                                                                unsigned long long n_rows, int passes, int dbits,
                                                                unsigned* __restrict__ block_hist,
                                                                unsigned* __restrict__ zero_from, size_t zero_words,
                                                                int* __restrict__ pair_seg, int* err,
                                                                unsigned* abort_word, unsigned abort_init,
                                                                int* __restrict__ n_uniq) {
  extern __shared__ unsigned lds_hist[];  // [passes][bins]
  const int bins = 1 << dbits;
  const unsigned mask = (unsigned)bins - 1u;
  const int lane = threadIdx.x & 63;
  for (int i = threadIdx.x; i < passes * bins; i += kAuxThreads) lds_hist[i] = 0;
  for (size_t i = (size_t)blockIdx.x * kAuxThreads + threadIdx.x; i < zero_words; i += (size_t)gridDim.x * kAuxThreads)
    zero_from[i] = &zero_from[i] == abort_word ? abort_init : 0u;  // (abort_init != 0: a test asks for a plan that gives up)
  // n_uniq ends as the smallest value anybody writes: the number of distinct ids, or -1 from a workgroup that gave up
  if (blockIdx.x == 0 && threadIdx.x == 0) *n_uniq = 0x7fffffff;
  __syncthreads();
  int bad = 0;
  const size_t tile_base = (size_t)blockIdx.x * tile_len;
  const size_t tile_end = tile_base + tile_len < (size_t)n ? tile_base + tile_len : (size_t)n;
  for (size_t base = tile_base; base < tile_end; base += (size_t)kAuxThreads * kHistBatch) {
    long long id[kHistBatch];
#pragma unroll
    for (int u = 0; u < kHistBatch; ++u) {  // all requests of the batch before the first use
      const size_t p = base + (size_t)u * kAuxThreads + threadIdx.x;
      id[u] = p < tile_end ? idx[p] : 0;
    }
#pragma unroll
    for (int u = 0; u < kHistBatch; ++u) {
      const size_t p = base + (size_t)u * kAuxThreads + threadIdx.x;
      const bool valid = p < tile_end;
      const unsigned key = clamp_id(id[u], n_rows, bad);
      for (int s = 0; s < passes; ++s) count_digit(lds_hist + s * bins, (key >> (s * dbits)) & mask, valid, lane);
      if (valid && pair_seg) pair_seg[p] = 0;  // "not alone"; the emit kernel overwrites the entries of one-pair segments
    }
  }
  if (bad && err) *err = 1;
  __syncthreads();
  for (int i = threadIdx.x; i < passes * bins; i += kAuxThreads)
    block_hist[(size_t)blockIdx.x * passes * bins + i] = lds_hist[i];
}

// digit_count[pass][digit] = sum over the tiles; one workgroup per (pass, 64 digits), its sixteen wavefronts take
// one stretch of the tiles each.  For the first pass the running sum is kept as well:
// tile_before[tile][digit] = ids with that digit in the tiles before it.
__global__ __launch_bounds__(kAuxThreads) void sort_sum_kernel(const unsigned* __restrict__ block_hist, int blocks,
                                                               int passes, int dbits,
                                                               unsigned* __restrict__ digit_count,
                                                               unsigned* __restrict__ tile_before) {
  __shared__ unsigned part[kAuxWaves][64];
  const int bins = 1 << dbits;
  const int groups = (bins + 63) / 64;
  const int s = blockIdx.x / groups;
  const int lane = threadIdx.x & 63;
  const int d = (blockIdx.x - s * groups) * 64 + lane;
  const int w = threadIdx.x >> 6;
  const int per_wave = (blocks + kAuxWaves - 1) / kAuxWaves;
  const int b_lo = w * per_wave, b_hi = min(blocks, b_lo + per_wave);
  const unsigned* src = block_hist + (size_t)s * bins + (d < bins ? d : 0);
  const size_t stride = (size_t)passes * bins;
  unsigned sum = 0;
  for (int b0 = b_lo; b0 < b_hi; b0 += 8) {
    unsigned v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = b0 + u < b_hi ? src[(size_t)(b0 + u) * stride] : 0u;
#pragma unroll
    for (int u = 0; u < 8; ++u) sum += v[u];
  }
  part[w][lane] = sum;
  __syncthreads();
  unsigned before = 0, all = 0;
#pragma unroll
  for (int i = 0; i < kAuxWaves; ++i) {
    const unsigned t = part[i][lane];
    before += i < w ? t : 0u;
    all += t;
  }
  if (d >= bins) return;
  if (w == 0) digit_count[s * bins + d] = all;
  if (s != 0) return;
  for (int b0 = b_lo; b0 < b_hi; b0 += 8) {
    unsigned v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = b0 + u < b_hi ? src[(size_t)(b0 + u) * stride] : 0u;
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      if (b0 + u < b_hi) tile_before[(size_t)(b0 + u) * bins + d] = before;
      before += v[u];
    }
  }
}

// ---- one radix pass -----------------------------------------------------------------------------
struct SortPassArgs {
  const long long* idx;             // IN_IDX: the ids; the payload is the position
  const unsigned long long* in;     // else: (key << 32 | payload) elements of the previous pass
  unsigned long long* out;          // packed output, or
  unsigned* out_keys;               // OUT_SPLIT: sorted ids and
  int* out_vals;                    //            pair positions as two arrays
  int n;
  int rounds;                       // elements per thread; a tile has rounds * NW * 64 elements
  int shift, dbits;
  size_t stage_bytes;               // LDS bytes of the region shared by the per-wavefront counters and the staged tile
  const unsigned* digit_count;      // [bins] of this pass: elements per digit in the whole input
  const unsigned* tile_before;      // IN_IDX: [tiles][bins] elements per digit in the tiles before each (from the sum kernel)
  // look-back tables of the other passes, each word = ready flag | count per digit:
  unsigned* level[3];               // [tiles / 16^l][bins], l = 0: one tile, 1: a group of 16 tiles, 2: 256 tiles
  unsigned* pre;                    // [tiles / 4096][bins]: everything up to the end of a stretch of 4096 tiles
  unsigned* ticket;
  unsigned* abort_flag;
  unsigned long long n_rows;
  int* err;
  unsigned spin_limit;
};

// Digits are owned by threads: thread t owns digit t (and t + threads when there are more digits
// than threads).
template <int NW, int MAXR, bool IN_IDX, bool OUT_SPLIT>
__global__ __launch_bounds__(NW * 64, (MAXR <= 8 ? 8 : 4)) void sort_pass_kernel(SortPassArgs A) {
  constexpr int NT = NW * 64;
  constexpr int PER = (1 << kSortMaxDigitBits) / NT > 1 ? (1 << kSortMaxDigitBits) / NT : 1;  // digits per thread, at most
  extern __shared__ __align__(16) unsigned char smem[];
  const int bins = 1 << A.dbits;
  const unsigned mask = (unsigned)bins - 1u;
  unsigned* counters = reinterpret_cast<unsigned*>(smem);                     // [waves][bins] while ranking
  unsigned long long* stage = reinterpret_cast<unsigned long long*>(smem);    // [tile] afterwards
  unsigned* local_base = reinterpret_cast<unsigned*>(smem + A.stage_bytes);   // [bins]
  unsigned* run_base = local_base + bins;                                     // [bins]
  unsigned* tmp = run_base + bins;                                            // 32 words
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int R = A.rounds;

  if (tid == 0) tmp[20] = atomicAdd(A.ticket, 1u);
  for (int d = lane; d < bins; d += 64) counters[w * bins + d] = 0;  // the wavefront's own row
  __syncthreads();
  const unsigned tile = tmp[20];
  const size_t tile_base = (size_t)tile * R * NT;
  const size_t wave_base = tile_base + (size_t)w * R * 64;
  const size_t n = (size_t)A.n;

  // 1. the tile's elements: wavefront w owns R * 64 consecutive ones, round r is 64 consecutive
  unsigned long long e[MAXR];
  int bad = 0;
#pragma unroll
  for (int r = 0; r < MAXR; ++r) {
    e[r] = ~0ull;
    if (r < R) {
      const size_t pos = wave_base + (size_t)r * 64 + lane;
      if (pos < n) {
        if constexpr (IN_IDX)
          e[r] = ((unsigned long long)clamp_id(A.idx[pos], A.n_rows, bad) << 32) | (unsigned)pos;
        else
          e[r] = A.in[pos];
      }
    }
  }
  (void)bad;  // the hist kernel has already reported ids outside the table

  // 2. rank inside the wavefront: position among the wavefront's elements with the same digit
  unsigned rank[MAXR];
#pragma unroll
  for (int r = 0; r < MAXR; ++r) {
    rank[r] = 0;
    if (r < R) {  // uniform
      const bool valid = wave_base + (size_t)r * 64 + lane < n;
      const unsigned d = ((unsigned)(e[r] >> 32) >> A.shift) & mask;
      const unsigned long long same = match_digit(d, A.dbits, __ballot(valid));
      const unsigned below = lanes_below(same);
      unsigned prev = 0;
      if (valid) prev = counters[w * bins + d];
      wave_lds_fence();  // every lane has read before the first lane of each digit writes
      if (valid && below == 0) counters[w * bins + d] = prev + (unsigned)__popcll(same);
      wave_lds_fence();
      rank[r] = prev + below;
    }
  }
  __syncthreads();

  // 3. per digit: the tile's count (published), and the wavefronts' rows turned into exclusive prefixes
  unsigned mine[PER], lb[PER], db[PER];
#pragma unroll
  for (int u = 0; u < PER; ++u) {
    const int d = tid + u * NT;
    mine[u] = 0;
    if (d < bins) {
      unsigned run = 0;
#pragma unroll
      for (int ww = 0; ww < NW; ++ww) {
        const unsigned t = counters[ww * bins + d];
        counters[ww * bins + d] = run;
        run += t;
      }
      mine[u] = run;
      if constexpr (!IN_IDX) st_agent(&A.level[0][(size_t)tile * bins + d], run | kReady);
    }
  }
  // position of a digit's first element inside the reordered tile, and in the whole output
  {
    unsigned carry_l = 0, carry_g = 0;
#pragma unroll
    for (int u = 0; u < PER; ++u) {  // digits [u * NT, (u + 1) * NT) in thread order
      const int d = tid + u * NT;
      unsigned tl = 0, tg = 0;
      lb[u] = carry_l + block_excl_scan<NW>(mine[u], tmp, &tl);
      db[u] = carry_g + block_excl_scan<NW>(d < bins ? A.digit_count[d] : 0u, tmp, &tg);
      carry_l += tl;
      carry_g += tg;
    }
  }

  // 4. elements with a digit in the tiles before this one.  The first pass has them from the sum kernel.  The
  // others look back: tiles form groups of 16, groups form blocks of 16 groups, and so on; a thread fetches,
  // per level, at most 15 independent words (the units of that level before its own inside the next-larger
  // unit), and the last tile of a unit publishes the unit's total as soon as it has it.  Beyond 4096 tiles a
  // chain of prefixes takes over.
#pragma unroll
  for (int u = 0; u < PER; ++u) {
    const int d = tid + u * NT;
    if (d < bins) {
      unsigned before = 0;
      [[maybe_unused]] unsigned gave_up = 0;  // (the mark on the device is what counts here)
      if constexpr (IN_IDX) {
        before = A.tile_before[(size_t)tile * bins + d];
      } else {
        unsigned unit = tile;  // my unit's number at this level
#pragma unroll
        for (int l = 0; l < 3; ++l) {
          const unsigned first = unit & ~(unsigned)(kGroup - 1);
          const unsigned* tab = A.level[l] + d;
          unsigned v[kGroup - 1];
#pragma unroll
          for (int j = 0; j < kGroup - 1; ++j) v[j] = first + j < unit ? ld_agent(tab + (size_t)(first + j) * bins) : kReady;
          unsigned here = 0;
#pragma unroll
          for (int j = 0; j < kGroup - 1; ++j) {
            if (first + j < unit) v[j] = wait_ready(tab + (size_t)(first + j) * bins, v[j], A.abort_flag, A.err, A.spin_limit, gave_up);
            here += v[j] & kCount;
          }
          before += here;
          // the last tile of a unit of the next level publishes that unit's total: everything before me
          // inside it (levels up to here) plus my own count
          const unsigned span = 1u << (4 * (l + 1));
          if ((tile & (span - 1)) == span - 1) {
            if (l < 2) st_agent(A.level[l + 1] + (size_t)(tile / span) * bins + d, ((before + mine[u]) & kCount) | kReady);
          }
          unit >>= 4;
        }
        if (tile >= 4096u) {
          const unsigned* p = &A.pre[(size_t)(tile / 4096u - 1) * bins + d];
          before += wait_ready(p, ld_agent(p), A.abort_flag, A.err, A.spin_limit, gave_up) & kCount;
        }
        if ((tile & 4095u) == 4095u) st_agent(&A.pre[(size_t)(tile / 4096u) * bins + d], ((before + mine[u]) & kCount) | kReady);
      }
      local_base[d] = lb[u];
      run_base[d] = db[u] + before - lb[u];  // + position in the reordered tile = global position
    }
  }
  // (A tile that gave up waiting has taken the missing counts as zero: its positions are wrong but inside the
  // output, like those of the tiles that read what it publishes; the emit kernel sees the mark and declares the
  // plan invalid, so nobody reads the result.)
  __syncthreads();

  // 5. position of every element in the tile reordered by digit
#pragma unroll
  for (int r = 0; r < MAXR; ++r) {
    if (r < R) {
      const unsigned d = ((unsigned)(e[r] >> 32) >> A.shift) & mask;
      if (wave_base + (size_t)r * 64 + lane < n) rank[r] += local_base[d] + counters[w * bins + d];
    }
  }
  __syncthreads();  // the counters are dead: their LDS becomes the staged tile
#pragma unroll
  for (int r = 0; r < MAXR; ++r) {
    if (r < R) {
      if (wave_base + (size_t)r * 64 + lane < n) stage[rank[r]] = e[r];
    }
  }
  __syncthreads();

  // 6. write the tile out in digit runs
  const size_t left = n - tile_base;  // tile_base < n: the grid has ceil(n / tile) tiles
  const int here = (int)(left < (size_t)R * NT ? left : (size_t)R * NT);
  for (int j = tid; j < here; j += NT) {
    const unsigned long long el = stage[j];
    const unsigned d = ((unsigned)(el >> 32) >> A.shift) & mask;
    const unsigned pos = run_base[d] + (unsigned)j;
    if constexpr (OUT_SPLIT) {
      A.out_keys[pos] = (unsigned)(el >> 32);
      A.out_vals[pos] = (int)(unsigned)el;
    } else {
      A.out[pos] = el;
    }
  }
}

// ---- emit ---------------------------------------------------------------------------------------
struct EmitArgs {
  const unsigned* sorted_ids;
  const int* order;
  int n;
  unsigned long long n_rows;
  int* seg_of_pos;
  long long* uniq;
  int* seg_start;
  long long* inverse;  // may be null
  int* pair_seg;       // may be null
  int* n_uniq;
  unsigned* agg;       // [tiles]: ready flag | segment heads in the tile
  unsigned* pre;       // [tiles / kEmitSuper]: ready flag | heads up to the end of a super-block
  unsigned* ticket;
  unsigned* abort_flag;
  int* err;
  unsigned spin_limit;
};

// Sorted positions per thread of the emit kernel: 16 for millions of positions (every tile pays the same fixed
// latencies -- look-back, scattered stores --, so fewer, longer tiles win there), fewer for short inputs, whose few
// long tiles would leave most of the chip idle (65,536 positions: 4 tiles of 16 rows took 16 us).  Measured plan
// times: 4.19 M positions 0.32 / 0.17 / 0.17 ms with 1 / 4 / 16 per thread; 1 M: 0.13 / 0.10 / 0.11; 524 k: 0.080 / 0.077 /
// 0.090; 262 k: 0.071 with 1 against 0.087 with 16.
static int emit_iters(size_t n) { return n <= ((size_t)1 << 18) ? 1 : (n <= ((size_t)1 << 20) ? 4 : kEmitIters); }

// Consecutive lanes own consecutive sorted positions (ITERS rows of 1024 per tile).  Segment
// numbers need the number of segment heads before the tile: look-back over the tiles' head counts as
// in the radix passes, one value per tile, read by the first wavefront.
template <int ITERS>
__global__ __launch_bounds__(kAuxThreads) void plan_emit_kernel(EmitArgs A) {
  constexpr int kEmitTile = kAuxThreads * ITERS;
  constexpr int kCounts = ITERS * kAuxWaves;            // 16, 64 or 256
  constexpr int kPerLane = kCounts >= 64 ? kCounts / 64 : 1;
  __shared__ unsigned counts[kCounts];  // heads per (iteration, wavefront), then their exclusive prefix
  __shared__ unsigned tmp[32];
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  if (tid == 0) tmp[20] = atomicAdd(A.ticket, 1u);
  __syncthreads();
  const unsigned tile = tmp[20];
  const long long n = A.n;
  const long long base = (long long)tile * kEmitTile;

  unsigned key[ITERS];
  unsigned heads = 0, singles = 0;  // bit it: my position of iteration it starts a segment / is a whole segment
  unsigned char below[ITERS];  // heads at lower lanes of my wavefront in the same iteration
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const long long p = base + it * kAuxThreads + tid;
    key[it] = p < n ? A.sorted_ids[p] : 0u;
    const unsigned prev = (p > 0 && p < n) ? A.sorted_ids[p - 1] : 0u;
    const unsigned next = p + 1 < n ? A.sorted_ids[p + 1] : 0u;
    const bool head = p < n && (p == 0 || prev != key[it]);
    const bool single = head && (p == n - 1 || next != key[it]) && (unsigned long long)key[it] < A.n_rows;
    heads |= (head ? 1u : 0u) << it;
    singles |= (single ? 1u : 0u) << it;
    const unsigned long long b = __ballot(head);
    below[it] = (unsigned char)lanes_below(b);
    if (lane == 0) counts[it * kAuxWaves + w] = (unsigned)__popcll(b);
  }
  __syncthreads();
  // exclusive prefix over the (iteration, wavefront) counts, in that order: kCounts values, kPerLane per lane
  if (w == 0) {
    unsigned c[kPerLane], s = 0;
#pragma unroll
    for (int i = 0; i < kPerLane; ++i) {
      c[i] = lane * kPerLane + i < kCounts ? counts[lane * kPerLane + i] : 0u;
      s += c[i];
    }
    unsigned inc = s;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const unsigned t = __shfl_up(inc, off);
      if (lane >= off) inc += t;
    }
    unsigned run = inc - s;
#pragma unroll
    for (int i = 0; i < kPerLane; ++i) {
      if (lane * kPerLane + i < kCounts) counts[lane * kPerLane + i] = run;
      run += c[i];
    }
    const unsigned total = (unsigned)__builtin_amdgcn_readlane((int)inc, 63);
    if (lane == 0) st_agent(&A.agg[tile], total | kReady);

    // look-back: heads in the tiles before this one
    unsigned sum = 0;
    [[maybe_unused]] unsigned gave_up = 0;  // (the mark on the device is what counts here)
    const int first = (int)(tile & ~(unsigned)(kEmitSuper - 1));
    unsigned v[kEmitSuper / 64];
#pragma unroll
    for (int u = 0; u < kEmitSuper / 64; ++u) {
      const int j = (int)tile - 1 - lane - 64 * u;
      v[u] = j >= first ? ld_agent(&A.agg[j]) : kReady;
    }
#pragma unroll
    for (int u = 0; u < kEmitSuper / 64; ++u) {
      const int j = (int)tile - 1 - lane - 64 * u;
      if (j >= first) v[u] = wait_ready(&A.agg[j], v[u], A.abort_flag, A.err, A.spin_limit, gave_up);
      sum += v[u] & kCount;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
    if (lane == 0) {
      if (first > 0) {
        const unsigned* p = &A.pre[first / kEmitSuper - 1];
        sum += wait_ready(p, ld_agent(p), A.abort_flag, A.err, A.spin_limit, gave_up) & kCount;
      }
      if ((tile & (kEmitSuper - 1)) == kEmitSuper - 1) st_agent(&A.pre[tile / kEmitSuper], ((sum + total) & kCount) | kReady);
      tmp[21] = sum;
      tmp[22] = ld_agent(A.abort_flag);
    }
  }
  __syncthreads();
  if (tmp[22]) {  // a tile gave up waiting: segment numbers are not trustworthy, write nothing but "no plan"
    if (tid == 0) {
      atomicMin(A.n_uniq, -1);  // every kernel that reads the plan looks at this first and leaves
      if (A.err) *A.err = 2;
    }
    return;
  }
  const unsigned first_seg = tmp[21];

#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const long long p = base + it * kAuxThreads + tid;
    if (p < n) {
      const bool head = (heads >> it) & 1u;
      const int seg = (int)(first_seg + counts[it * kAuxWaves + w] + below[it] + (head ? 1u : 0u)) - 1;
      A.seg_of_pos[p] = seg;
      if (head) {
        A.uniq[seg] = (long long)key[it];
        A.seg_start[seg] = (int)p;
      }
      if (A.inverse) A.inverse[A.order[p]] = seg;
      if (A.pair_seg && ((singles >> it) & 1u)) A.pair_seg[A.order[p]] = seg | (int)0x80000000;  // sign bit + segment number
      if (p == n - 1) {  // the last position closes the list
        A.seg_start[seg + 1] = (int)n;
        atomicMin(A.n_uniq, seg + 1 - ((unsigned long long)key[it] >= A.n_rows ? 1 : 0));  // ids outside the table are not counted
      }
    }
  }
}


// ---- small inputs: the whole plan in one launch ---------------------------------------------------
// A step whose negatives are shared by the batch sorts K + B (+ anchors) ids, a couple of thousand: six dependent
// launches would cost more than the work.  One workgroup sorts the positions by id in LDS -- a stable LSD radix
// sort with digits of up to 7 bits, ranked inside a wavefront with one ballot per bit as in the radix passes above,
// every wavefront owning a contiguous stretch of the list -- and writes every array of the plan.
// (A bitonic network over 64-bit (id, position) keys took 22 us for 1,536 ids: 66 stages, each a barrier across
// sixteen wavefronts; the radix sort has three barriers per pass and four passes for a 25-bit id.)
constexpr int kSmallPlanMax = 4096;
constexpr int kSmallThreads = 1024;
constexpr int kSmallWaves = kSmallThreads / 64;
constexpr int kSmallDigitBits = 7;
constexpr int kSmallBins = 1 << kSmallDigitBits;
constexpr int kSmallRounds = kSmallPlanMax / kSmallThreads;  // positions per thread, at most

// LDS: keys [n] (32-bit ids, by original position), then two lists of positions [n] (16-bit), used in turn
__global__ __launch_bounds__(kSmallThreads) void plan_small_kernel(const long long* __restrict__ idx, int n, int passes,
                                                                 int dbits, unsigned long long n_rows,
                                                                 int* __restrict__ order,
                                                                 unsigned* __restrict__ sorted_ids,
                                                                 int* __restrict__ seg_of_pos, long long* __restrict__ uniq,
                                                                 int* __restrict__ seg_start, long long* __restrict__ inverse,
                                                                 int* __restrict__ pair_seg, int* __restrict__ n_uniq,
                                                                 int* err) {
  extern __shared__ unsigned small_lds[];
  __shared__ unsigned cnt[kSmallWaves * kSmallBins];  // per wavefront and digit: elements so far, then the prefix over wavefronts
  __shared__ unsigned dig_base[kSmallBins];
  __shared__ unsigned tmp[32];
  const int n_even = (n + 1) & ~1;
  unsigned* keys = small_lds;
  unsigned short* list_a = reinterpret_cast<unsigned short*>(small_lds + n_even);
  unsigned short* list_b = list_a + n_even;
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  int bad = 0;
  for (int i = tid; i < n; i += kSmallThreads) {
    keys[i] = clamp_id(idx[i], n_rows, bad);
    list_a[i] = (unsigned short)i;
  }
  if (bad && err) *err = 1;
  const int bins = 1 << dbits;
  const unsigned mask = (unsigned)bins - 1u;
  // wavefront w owns positions [w * per_wave, (w + 1) * per_wave) of the current list, 64 at a time
  const int rounds = (n + kSmallThreads - 1) / kSmallThreads;
  const int per_wave = rounds * 64;
  unsigned short* src = list_a;
  unsigned short* dst = list_b;
  for (int pass = 0; pass < passes; ++pass) {
    const int shift = pass * dbits;
    for (int i = tid; i < kSmallWaves * bins; i += kSmallThreads) cnt[i] = 0u;
    __syncthreads();
    unsigned el[kSmallRounds], rank[kSmallRounds], dig[kSmallRounds];
#pragma unroll
    for (int r = 0; r < kSmallRounds; ++r) {
      el[r] = rank[r] = dig[r] = 0u;
      if (r < rounds) {  // uniform
        const int p = w * per_wave + r * 64 + lane;
        const bool valid = p < n;
        if (valid) el[r] = src[p];
        const unsigned d = valid ? (keys[el[r]] >> shift) & mask : 0u;
        dig[r] = d;
        const unsigned long long same = match_digit(d, dbits, __ballot(valid));
        const unsigned below = lanes_below(same);
        unsigned prev = 0;
        if (valid) prev = cnt[w * bins + d];
        wave_lds_fence();  // every lane has read before the first lane of each digit writes
        if (valid && below == 0) cnt[w * bins + d] = prev + (unsigned)__popcll(same);
        wave_lds_fence();
        rank[r] = prev + below;
      }
    }
    __syncthreads();
    unsigned total = 0;
    if (tid < bins) {
      unsigned run = 0;
#pragma unroll
      for (int ww = 0; ww < kSmallWaves; ++ww) {
        const unsigned t = cnt[ww * bins + tid];
        cnt[ww * bins + tid] = run;
        run += t;
      }
      total = run;
    }
    const unsigned base = block_excl_scan<kSmallWaves>(total, tmp, nullptr);
    if (tid < bins) dig_base[tid] = base;
    __syncthreads();
#pragma unroll
    for (int r = 0; r < kSmallRounds; ++r) {
      if (r < rounds && w * per_wave + r * 64 + lane < n)
        dst[dig_base[dig[r]] + cnt[w * bins + dig[r]] + rank[r]] = (unsigned short)el[r];
    }
    unsigned short* t = src;
    src = dst;
    dst = t;
    __syncthreads();  // the new list is complete, and nobody reads the counters any more
  }
  // segment heads and numbers, one sorted position per thread at a time
  unsigned carry = 0;
  for (int base = 0; base < n; base += kSmallThreads) {
    const int p = base + tid;
    const bool in = p < n;
    const int pair = in ? (int)src[p] : 0;
    const unsigned key = in ? keys[pair] : 0u;
    const bool head = in && (p == 0 || keys[src[p - 1]] != key);
    const bool last_of_seg = in && (p == n - 1 || keys[src[p + 1]] != key);
    unsigned total = 0;
    const unsigned before = block_excl_scan<kSmallWaves>(head ? 1u : 0u, tmp, &total);
    if (in) {
      const int seg = (int)(carry + before + (head ? 1u : 0u)) - 1;
      order[p] = pair;
      sorted_ids[p] = key;
      seg_of_pos[p] = seg;
      if (head) {
        uniq[seg] = (long long)key;
        seg_start[seg] = p;
      }
      if (inverse) inverse[pair] = seg;
      if (pair_seg) pair_seg[pair] = (head && last_of_seg && (unsigned long long)key < n_rows) ? (seg | (int)0x80000000) : 0;
      if (p == n - 1) {
        seg_start[seg + 1] = n;
        *n_uniq = seg + 1 - ((unsigned long long)key >= n_rows ? 1 : 0);  // ids outside the table are not counted
      }
    }
    carry += total;
  }
}

// ---- host side ----------------------------------------------------------------------------------
static unsigned key_bits(size_t n_values) {
  unsigned bits = 1;
  while (bits < 32 && (1ull << bits) < n_values) ++bits;
  return bits;
}

// LDS bytes a workgroup may use on the current device (gfx950: 160 KiB); 64 KiB when it cannot be asked.
static size_t lds_limit() {
  static std::mutex mu;
  static size_t per_device[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 64 * 1024;
  std::lock_guard<std::mutex> lock(mu);
  if (!per_device[dev]) {
    int v = 0;
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) != hipSuccess || v <= 0) v = 64 * 1024;
    per_device[dev] = (size_t)v;
  }
  return per_device[dev];
}

// Wavefronts per workgroup of the radix passes.  Measured on MI355X (4M pairs, 27-bit ids): 16 wavefronts
// with 16 elements per thread, one workgroup per CU, 36 us per pass; smaller workgroups or tiles are
// slower (47-56 us), the cost per tile being dominated by the look-back and the workgroup-wide steps.
constexpr int kSortWaves = 16;

struct PlanLayout {
  int passes, dbits, bins, nw, rounds, tiles, units[3], chain, hist_blocks, emit_tiles, emit_supers;
  size_t stage_bytes, pass_lds;
  size_t a_off, b_off, bh_off, count_off, tb_off, zero_off, zero_words, total;
  // inside the zeroed region (in words from zero_off)
  size_t level_w[3], pre_w, eagg_w, epre_w, ticket_w, abort_w;
};

static PlanLayout plan_layout(size_t n, size_t n_rows) {
  auto up = [](size_t x) { return (x + 255) & ~(size_t)255; };
  PlanLayout L{};
  const unsigned bits = key_bits(n_rows + 1);  // + the key of ids outside the table
  L.passes = (int)((bits + kSortMaxDigitBits - 1) / kSortMaxDigitBits);
  L.dbits = (int)((bits + L.passes - 1) / L.passes);
  L.bins = 1 << L.dbits;
  L.nw = kSortWaves;
  const size_t nt = (size_t)L.nw * 64;
  // elements per thread: enough tiles to fill the chip (one workgroup per CU), tiles as large as the LDS allows
  const size_t fixed_lds = (size_t)(2 * L.bins + 32) * sizeof(unsigned);
  const size_t counters = (size_t)L.nw * L.bins * sizeof(unsigned);
  const size_t per_cu = 16 / (size_t)L.nw;  // workgroups that share a CU's LDS
  size_t max_rounds = (lds_limit() / per_cu - fixed_lds - 1024) / (nt * 8);
  if (max_rounds > (size_t)kSortMaxRounds) max_rounds = kSortMaxRounds;
  if (max_rounds < 1) max_rounds = 1;
  size_t rounds = (n + nt * 256 * per_cu - 1) / (nt * 256 * per_cu);
  if (rounds < 1) rounds = 1;
  if (rounds > max_rounds) rounds = max_rounds;
  L.rounds = (int)rounds;
  const size_t tile = rounds * nt;
  L.tiles = (int)((n + tile - 1) / tile);
  L.units[0] = L.tiles;
  L.units[1] = (L.tiles + kGroup - 1) / kGroup;
  L.units[2] = (L.units[1] + kGroup - 1) / kGroup;
  L.chain = (L.tiles + 4095) / 4096;
  L.stage_bytes = tile * 8 > counters ? tile * 8 : counters;
  L.pass_lds = L.stage_bytes + fixed_lds;
  L.hist_blocks = L.tiles;  // the hist kernel counts per tile of the radix passes
  const size_t emit_tile = (size_t)kAuxThreads * emit_iters(n);
  L.emit_tiles = (int)((n + emit_tile - 1) / emit_tile);
  L.emit_supers = (L.emit_tiles + kEmitSuper - 1) / kEmitSuper;
  L.a_off = 0;
  L.b_off = up(n * 8);
  L.bh_off = L.b_off + (L.passes > 2 ? up(n * 8) : 0);
  L.count_off = L.bh_off + up((size_t)L.hist_blocks * L.passes * L.bins * 4);
  L.tb_off = L.count_off + up((size_t)L.passes * L.bins * 4);
  L.zero_off = L.tb_off + up((size_t)L.tiles * L.bins * 4);
  size_t wds = 0;
  for (int l = 0; l < 3; ++l) {
    L.level_w[l] = wds;
    wds += (size_t)L.passes * L.units[l] * L.bins;
  }
  L.pre_w = wds;    wds += (size_t)L.passes * L.chain * L.bins;
  L.eagg_w = wds;   wds += (size_t)L.emit_tiles;
  L.epre_w = wds;   wds += (size_t)L.emit_supers;
  L.ticket_w = wds; wds += (size_t)L.passes + 1;
  L.abort_w = wds;  wds += 1;
  L.zero_words = wds;
  L.total = L.zero_off + up(wds * 4);
  return L;
}

template <int NW, int MAXR, bool IN_IDX, bool OUT_SPLIT>
static void launch_pass(hipStream_t st, const PlanLayout& L, const SortPassArgs& A) {
  auto kernel = sort_pass_kernel<NW, MAXR, IN_IDX, OUT_SPLIT>;
  // More than 64 KiB of dynamic LDS: said once per kernel and device (not again under a later stream
  // capture); a runtime that does not know the attribute leaves it to the launch to accept or refuse the size.
  if (L.pass_lds > 64 * 1024) {
    static std::mutex mu;
    static bool told[64] = {};
    int dev = 0;
    if (hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < 64) {
      std::lock_guard<std::mutex> lock(mu);
      if (!told[dev]) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                  (int)lds_limit());
        (void)hipGetLastError();
        told[dev] = true;
      }
    }
  }
  hipLaunchKernelGGL(kernel, dim3((unsigned)L.tiles), dim3(NW * 64), L.pass_lds, st, A);
}

template <int NW, int MAXR>
static void launch_pass_r(hipStream_t st, const PlanLayout& L, const SortPassArgs& A, bool first, bool last) {
  if (first && last) launch_pass<NW, MAXR, true, true>(st, L, A);
  else if (first) launch_pass<NW, MAXR, true, false>(st, L, A);
  else if (last) launch_pass<NW, MAXR, false, true>(st, L, A);
  else launch_pass<NW, MAXR, false, false>(st, L, A);
}
template <int NW>
static void launch_pass_nw(hipStream_t st, const PlanLayout& L, const SortPassArgs& A, bool first, bool last) {
  // (a step of B x (1 + K) pairs -- positives beside the negatives -- lies just beyond 256 tiles of 16 elements
  // per thread and still fits one tile per CU with 17: the third form saves such steps a second round of
  // workgroups, 51 -> 37 us per pass at 4.2 M pairs, at the price of a few spilled registers)
  if (L.rounds <= 8) launch_pass_r<NW, 8>(st, L, A, first, last);
  else if (L.rounds <= 16) launch_pass_r<NW, 16>(st, L, A, first, last);
  else launch_pass_r<NW, kSortMaxRounds>(st, L, A, first, last);
}

}  // namespace smx

extern "C" {

size_t smx_plan_workspace_bytes(size_t n_pairs, size_t n_rows) {
  if (n_pairs == 0) return 256;
  if (n_pairs > 0x7fffffffull || n_rows == 0 || n_rows > 0xffffffffull) return 0;
  return smx::plan_layout(n_pairs, n_rows).total;
}

}  // extern "C"

namespace smx {

// spin_limit, force_abort: kSpinLimit and 0 for every caller but the measuring entry point
static int plan_build(void* stream, const int64_t* idx, size_t n_pairs, size_t n_rows, void* workspace,
                      size_t workspace_bytes, int32_t* order, int32_t* sorted_ids, int32_t* seg_of_pos, int64_t* uniq,
                      int32_t* seg_start, int64_t* inverse, int32_t* pair_seg, int32_t* n_uniq, int* err_flag,
                      unsigned spin_limit, int force_abort) {
  if (!idx || !order || !sorted_ids || !seg_of_pos || !uniq || !seg_start || !n_uniq || !workspace)
    return fail(SMX_ERR_ARG, "null pointer in plan build");
  if (n_pairs == 0 || n_pairs > 0x7fffffffull) return fail(SMX_ERR_SHAPE, "pair count %zu out of range", n_pairs);
  if (n_rows == 0 || n_rows > 0xffffffffull) return fail(SMX_ERR_SHAPE, "entity count %zu needs ids wider than 32 bits", n_rows);
  if (n_pairs <= (size_t)kSmallPlanMax && !force_abort) {
    const unsigned bits = key_bits(n_rows + 1);  // + the key of ids outside the table
    const int passes = (int)((bits + kSmallDigitBits - 1) / kSmallDigitBits);
    const int dbits = (int)((bits + passes - 1) / passes);
    const size_t n_even = (n_pairs + 1) & ~(size_t)1;
    hipLaunchKernelGGL(plan_small_kernel, dim3(1), dim3(kSmallThreads), n_even * (sizeof(unsigned) + 2 * sizeof(unsigned short)),
                       as_stream(stream), reinterpret_cast<const long long*>(idx), (int)n_pairs, passes, dbits,
                       (unsigned long long)n_rows, order, reinterpret_cast<unsigned*>(sorted_ids), seg_of_pos,
                       reinterpret_cast<long long*>(uniq), seg_start, reinterpret_cast<long long*>(inverse), pair_seg,
                       n_uniq, err_flag);
    return check_launch("plan build (one workgroup)");
  }
  const PlanLayout L = plan_layout(n_pairs, n_rows);
  if (workspace_bytes < L.total)
    return fail(SMX_ERR_WORKSPACE, "plan workspace too small: %zu < %zu", workspace_bytes, L.total);
  if (reinterpret_cast<uintptr_t>(workspace) & 255u) return fail(SMX_ERR_ARG, "workspace must be 256-byte aligned");
  if (L.pass_lds > lds_limit())
    return fail(SMX_ERR_HIP, "a radix pass needs %zu bytes of LDS per workgroup, the device allows %zu", L.pass_lds, lds_limit());
  hipStream_t st = as_stream(stream);
  char* ws = static_cast<char*>(workspace);
  unsigned long long* buf_a = reinterpret_cast<unsigned long long*>(ws + L.a_off);
  unsigned long long* buf_b = reinterpret_cast<unsigned long long*>(ws + L.b_off);
  unsigned* block_hist = reinterpret_cast<unsigned*>(ws + L.bh_off);
  unsigned* digit_count = reinterpret_cast<unsigned*>(ws + L.count_off);
  unsigned* tile_before = reinterpret_cast<unsigned*>(ws + L.tb_off);
  unsigned* zeroed = reinterpret_cast<unsigned*>(ws + L.zero_off);
  const int n = (int)n_pairs;

  hipLaunchKernelGGL(sort_hist_kernel, dim3((unsigned)L.hist_blocks), dim3(kAuxThreads),
                     (size_t)L.passes * L.bins * sizeof(unsigned), st, reinterpret_cast<const long long*>(idx), n,
                     L.rounds * L.nw * 64, (unsigned long long)n_rows, L.passes, L.dbits, block_hist, zeroed, L.zero_words, pair_seg,
                     err_flag,
                     zeroed + L.abort_w, force_abort ? 1u : 0u, n_uniq);
  hipLaunchKernelGGL(sort_sum_kernel, dim3((unsigned)(L.passes * ((L.bins + 63) / 64))), dim3(kAuxThreads), 0, st, block_hist,
                     L.hist_blocks, L.passes, L.dbits, digit_count, tile_before);
  for (int s = 0; s < L.passes; ++s) {
    SortPassArgs A{};
    const bool first = s == 0, last = s == L.passes - 1;
    // the packed buffers are used in turn; the last pass writes the plan's two arrays
    A.idx = reinterpret_cast<const long long*>(idx);
    A.in = (s % 2 == 1) ? buf_a : buf_b;
    A.out = (s % 2 == 0) ? buf_a : buf_b;
    A.out_keys = reinterpret_cast<unsigned*>(sorted_ids);
    A.out_vals = order;
    A.n = n;
    A.rounds = L.rounds;
    A.shift = s * L.dbits;
    A.dbits = L.dbits;
    A.stage_bytes = L.stage_bytes;
    A.digit_count = digit_count + (size_t)s * L.bins;
    A.tile_before = tile_before;
    for (int l = 0; l < 3; ++l) A.level[l] = zeroed + L.level_w[l] + (size_t)s * L.units[l] * L.bins;
    A.pre = zeroed + L.pre_w + (size_t)s * L.chain * L.bins;
    A.ticket = zeroed + L.ticket_w + s;
    A.abort_flag = zeroed + L.abort_w;
    A.n_rows = (unsigned long long)n_rows;
    A.err = err_flag;
    A.spin_limit = spin_limit;
    launch_pass_nw<kSortWaves>(st, L, A, first, last);
    if (int rc = check_launch("radix pass")) return rc;
  }
  EmitArgs E{};
  E.sorted_ids = reinterpret_cast<const unsigned*>(sorted_ids);
  E.order = order;
  E.n = n;
  E.n_rows = (unsigned long long)n_rows;
  E.seg_of_pos = seg_of_pos;
  E.uniq = reinterpret_cast<long long*>(uniq);
  E.seg_start = seg_start;
  E.inverse = reinterpret_cast<long long*>(inverse);
  E.pair_seg = pair_seg;
  E.n_uniq = n_uniq;
  E.agg = zeroed + L.eagg_w;
  E.pre = zeroed + L.epre_w;
  E.ticket = zeroed + L.ticket_w + L.passes;
  E.abort_flag = zeroed + L.abort_w;
  E.err = err_flag;
  E.spin_limit = spin_limit;
  switch (emit_iters(n_pairs)) {
    case 1: hipLaunchKernelGGL(plan_emit_kernel<1>, dim3((unsigned)L.emit_tiles), dim3(kAuxThreads), 0, st, E); break;
    case 4: hipLaunchKernelGGL(plan_emit_kernel<4>, dim3((unsigned)L.emit_tiles), dim3(kAuxThreads), 0, st, E); break;
    default: hipLaunchKernelGGL(plan_emit_kernel<kEmitIters>, dim3((unsigned)L.emit_tiles), dim3(kAuxThreads), 0, st, E);
  }
  return check_launch("plan build");
}

}  // namespace smx

extern "C" {

int smx_plan_build(void* stream, const int64_t* idx, size_t n_pairs, size_t n_rows, void* workspace,
                   size_t workspace_bytes, int32_t* order, int32_t* sorted_ids, int32_t* seg_of_pos, int64_t* uniq,
                   int32_t* seg_start, int64_t* inverse, int32_t* pair_seg, int32_t* n_uniq, int* err_flag) {
  return smx::plan_build(stream, idx, n_pairs, n_rows, workspace, workspace_bytes, order, sorted_ids, seg_of_pos, uniq,
                         seg_start, inverse, pair_seg, n_uniq, err_flag, smx::kSpinLimit, 0);
}

int smx_measure_plan_build(void* stream, const int64_t* idx, size_t n_pairs, size_t n_rows, void* workspace,
                           size_t workspace_bytes, int32_t* order, int32_t* sorted_ids, int32_t* seg_of_pos,
                           int64_t* uniq, int32_t* seg_start, int64_t* inverse, int32_t* pair_seg, int32_t* n_uniq,
                           int* err_flag, unsigned spin_limit, int force_abort) {
  return smx::plan_build(stream, idx, n_pairs, n_rows, workspace, workspace_bytes, order, sorted_ids, seg_of_pos, uniq,
                         seg_start, inverse, pair_seg, n_uniq, err_flag, spin_limit, force_abort);
}


}  // extern "C"

// ---- row gather -------------------------------------------------------------------------------
// out[k,:] = table[idx[k],:], one wavefront per row with 16-byte column loads when alignment allows.
// The plain lookup of the reference (smore/common/embedding/embed_rw.py:74-75) for callers that
// need the rows themselves (positives, anchors) rather than a fused score.
namespace smx {

template <int VEC>
__global__ __launch_bounds__(256) void gather_rows_kernel(const float* __restrict__ table,
                                                          const long long* __restrict__ idx, float* __restrict__ out,
                                                          int n, int ncol, unsigned long long n_rows, int* err) {
  const int lane = threadIdx.x & 63;
  const int k = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (k >= n) return;
  long long row = idx[k];
  if ((unsigned long long)row >= n_rows) {
    if (err && lane == 0) *err = 1;
    row = 0;
  }
  const size_t row_len = (size_t)ncol * VEC;
  for (int c = lane; c < ncol; c += 64) {
    if (VEC == 4) {  // the copy is written once and read by a later kernel: non-temporal store
      typedef float gvec4 __attribute__((ext_vector_type(4)));
      __builtin_nontemporal_store(reinterpret_cast<const gvec4*>(table + (size_t)row * row_len)[c],
                                  reinterpret_cast<gvec4*>(out + (size_t)k * row_len) + c);
    } else
      out[(size_t)k * row_len + c] = table[(size_t)row * row_len + c];
  }
}

}  // namespace smx

extern "C" int smx_gather_rows(void* stream, const float* table, size_t n_rows, size_t row_len, const int64_t* idx,
                               size_t n, float* out, int* err_flag) {
  using namespace smx;
  if (!table || !idx || !out) return fail(SMX_ERR_ARG, "null pointer in gather");
  if (n == 0 || n > 0x7fffffffull || row_len == 0 || row_len > 0x7fffffffull)
    return fail(SMX_ERR_SHAPE, "gather size out of range");
  hipStream_t st = as_stream(stream);
  const unsigned blocks = (unsigned)((n + 3) / 4);
  if (row_len % 4 == 0 && aligned16(table) && aligned16(out))
    hipLaunchKernelGGL(gather_rows_kernel<4>, dim3(blocks), dim3(256), 0, st, table,
                       reinterpret_cast<const long long*>(idx), out, (int)n, (int)(row_len / 4),
                       (unsigned long long)n_rows, err_flag);
  else
    hipLaunchKernelGGL(gather_rows_kernel<1>, dim3(blocks), dim3(256), 0, st, table,
                       reinterpret_cast<const long long*>(idx), out, (int)n, (int)row_len, (unsigned long long)n_rows,
                       err_flag);
  return check_launch("gather rows");
}
