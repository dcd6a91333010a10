// Segment plan: groups the (query, negative) pairs of one step by entity id.
//
// Replaces merge_grad_indices (smore/common/embedding/embed_optimizer.py:39-42),
// i.e. torch.unique(ids, return_inverse=True), which the reference runs on the
// host CPU, with a device pipeline:
//   keys  = (uint32) idx[p]                      narrow + range check
//   sort  (key, p) by key                        LSD radix sort, stable, only the
//                                                bits an id below n_rows can have
//   count heads (key[p] != key[p-1]) per span of 2048 positions, prefix over the spans,
//   emit  seg_of_pos, uniq, seg_start, inverse, n_uniq
// The sort is stable, so inside a segment pairs stay in ascending pair order:
// every later reduction over a segment has one fixed summation order.
#include <cstring>

#include <rocprim/device/device_radix_sort.hpp>
#include <rocprim/iterator/counting_iterator.hpp>

#include "smx_common.h"

namespace smx {

__global__ __launch_bounds__(256) void plan_keys_kernel(const long long* __restrict__ idx, unsigned* __restrict__ keys,
                                                        int* __restrict__ pair_seg, int n, unsigned long long n_rows,
                                                        int* err) {
  const int p = blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= n) return;
  if (pair_seg) pair_seg[p] = 0;  // "not alone"; the emit kernel overwrites the entries of one-pair segments
  long long id = idx[p];
  if ((unsigned long long)id >= n_rows) {
    if (err) *err = 1;
    id = 0;
  }
  keys[p] = (unsigned)id;
}

// Segment numbering without a device-wide scan primitive: every workgroup owns kPlanSpan consecutive
// sorted positions.  plan_count counts the segment heads of each span, plan_offsets (one workgroup)
// turns the counts into the number of the first segment of each span, and plan_emit recounts its span
// with a running prefix and writes the plan.  No workgroup waits for another one.
constexpr int kPlanIters = 8;
constexpr int kPlanSpan = 256 * kPlanIters;

__device__ __forceinline__ bool is_head(const int* __restrict__ sorted_ids, int p, int n) {
  return p < n && (p == 0 || sorted_ids[p] != sorted_ids[p - 1]);
}

__global__ __launch_bounds__(256) void plan_count_kernel(const int* __restrict__ sorted_ids, int n,
                                                         unsigned* __restrict__ span_heads) {
  __shared__ unsigned per_wave[4];
  const int base = blockIdx.x * kPlanSpan;
  unsigned cnt = 0;
#pragma unroll
  for (int it = 0; it < kPlanIters; ++it)
    cnt += (unsigned)__popcll(__ballot(is_head(sorted_ids, base + it * 256 + (int)threadIdx.x, n)));
  if ((threadIdx.x & 63) == 0) per_wave[threadIdx.x >> 6] = cnt;
  __syncthreads();
  if (threadIdx.x == 0) span_heads[blockIdx.x] = per_wave[0] + per_wave[1] + per_wave[2] + per_wave[3];
}

// exclusive prefix of span_heads -> span_first; also the segment count and the end marker of seg_start
__global__ __launch_bounds__(1024) void plan_offsets_kernel(const unsigned* __restrict__ span_heads,
                                                            unsigned* __restrict__ span_first, int spans,
                                                            int* __restrict__ n_uniq, int* __restrict__ seg_start, int n) {
  __shared__ unsigned buf[1024];
  __shared__ unsigned carry;
  if (threadIdx.x == 0) carry = 0;
  __syncthreads();
  for (int base = 0; base < spans; base += 1024) {
    const int i = base + (int)threadIdx.x;
    const unsigned mine = i < spans ? span_heads[i] : 0u;
    buf[threadIdx.x] = mine;
    __syncthreads();
    for (int step = 1; step < 1024; step <<= 1) {  // Hillis-Steele inclusive scan
      const unsigned add = threadIdx.x >= (unsigned)step ? buf[threadIdx.x - step] : 0u;
      __syncthreads();
      buf[threadIdx.x] += add;
      __syncthreads();
    }
    if (i < spans) span_first[i] = carry + buf[threadIdx.x] - mine;
    __syncthreads();
    if (threadIdx.x == 1023) carry += buf[1023];
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    *n_uniq = (int)carry;
    seg_start[carry] = n;
  }
}

__global__ __launch_bounds__(256) void plan_emit_kernel(const int* __restrict__ sorted_ids, const int* __restrict__ order,
                                                        const unsigned* __restrict__ span_first,
                                                        int* __restrict__ seg_of_pos, long long* __restrict__ uniq,
                                                        int* __restrict__ seg_start, long long* __restrict__ inverse,
                                                        int* __restrict__ pair_seg, int n) {
  __shared__ unsigned counts[kPlanIters][4];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int base = blockIdx.x * kPlanSpan;
  bool head[kPlanIters];
  unsigned below[kPlanIters];  // heads at lower lanes of this wavefront in the same iteration
#pragma unroll
  for (int it = 0; it < kPlanIters; ++it) {
    head[it] = is_head(sorted_ids, base + it * 256 + (int)threadIdx.x, n);
    const unsigned long long b = __ballot(head[it]);
    below[it] = (unsigned)__popcll(b & ((1ull << lane) - 1ull));
    if (lane == 0) counts[it][wave] = (unsigned)__popcll(b);
  }
  __syncthreads();
  unsigned running = span_first[blockIdx.x];
#pragma unroll
  for (int it = 0; it < kPlanIters; ++it) {
    unsigned before = running;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      if (w < wave) before += counts[it][w];
      running += counts[it][w];
    }
    const int p = base + it * 256 + (int)threadIdx.x;
    if (p < n) {
      const int seg = (int)(before + below[it] + (head[it] ? 1u : 0u)) - 1;
      seg_of_pos[p] = seg;
      if (head[it]) {
        uniq[seg] = (long long)(unsigned)sorted_ids[p];
        seg_start[seg] = p;
      }
      if (inverse) inverse[order[p]] = seg;
      if (pair_seg && head[it] && (p == n - 1 || sorted_ids[p + 1] != sorted_ids[p]))
        pair_seg[order[p]] = seg | (int)0x80000000;  // this pair is its segment: sign bit + segment number
    }
  }
}

static unsigned key_bits(size_t n_rows) {
  unsigned bits = 1;
  while (bits < 32 && (1ull << bits) < n_rows) ++bits;
  return bits;
}

// rocPRIM ships no tuned radix-sort configuration for gfx950 and falls back to 8-bit digits; measured
// on MI355X, one-sweep passes over 9-bit digits (10-bit when that saves a whole pass) sort the plan's
// (id, pair) list 1.2-2.4x faster: 27-bit ids of 4M pairs in 3 passes instead of 4, 20-bit ids in 2.
// Above 4096 pairs the one-sweep path is used instead of rocPRIM's merge sort (its default up to 1M).
using Sort9 = rocprim::radix_sort_config<
    rocprim::default_config, rocprim::default_config,
    rocprim::radix_sort_onesweep_config<rocprim::kernel_config<1024, 8>, rocprim::kernel_config<1024, 8>, 9,
                                        rocprim::block_radix_rank_algorithm::match>,
    4096>;
using Sort10 = rocprim::radix_sort_config<
    rocprim::default_config, rocprim::default_config,
    rocprim::radix_sort_onesweep_config<rocprim::kernel_config<1024, 4>, rocprim::kernel_config<1024, 4>, 10,
                                        rocprim::block_radix_rank_algorithm::match>,
    4096>;

static bool ten_bit_digits(unsigned bits) { return (bits + 9) / 10 < (bits + 8) / 9; }

static hipError_t sort_pairs(void* temp, size_t& temp_bytes, unsigned* keys, unsigned* keys_out, int* order, size_t n,
                             unsigned bits, hipStream_t st) {
  if (ten_bit_digits(bits))
    return rocprim::radix_sort_pairs<Sort10>(temp, temp_bytes, keys, keys_out, rocprim::counting_iterator<int>(0), order,
                                             n, 0, bits, st);
  return rocprim::radix_sort_pairs<Sort9>(temp, temp_bytes, keys, keys_out, rocprim::counting_iterator<int>(0), order, n,
                                          0, bits, st);
}

struct PlanScratch {
  size_t keys_off, heads_off, first_off, temp_off, temp_bytes, total;
  int spans;
};

static hipError_t plan_scratch(size_t n, size_t n_rows, PlanScratch* s) {
  size_t sort_bytes = 0;
  unsigned* kp = nullptr;
  int* ip = nullptr;
  hipError_t e = sort_pairs(nullptr, sort_bytes, kp, kp, ip, n, key_bits(n_rows), (hipStream_t)0);
  if (e != hipSuccess) return e;
  auto up = [](size_t x) { return (x + 255) & ~(size_t)255; };
  s->spans = (int)((n + kPlanSpan - 1) / kPlanSpan);
  s->keys_off = 0;
  s->heads_off = up(n * sizeof(unsigned));
  s->first_off = s->heads_off + up((size_t)s->spans * sizeof(unsigned));
  s->temp_off = s->first_off + up((size_t)s->spans * sizeof(unsigned));
  s->temp_bytes = up(sort_bytes);
  s->total = s->temp_off + s->temp_bytes;
  return hipSuccess;
}

}  // namespace smx

extern "C" {

size_t smx_plan_workspace_bytes(size_t n_pairs, size_t n_rows) {
  smx::PlanScratch s;
  if (n_pairs == 0) return 256;
  if (smx::plan_scratch(n_pairs, n_rows, &s) != hipSuccess) return 0;
  return s.total;
}

int smx_plan_build(void* stream, const int64_t* idx, size_t n_pairs, size_t n_rows, void* workspace,
                   size_t workspace_bytes, int32_t* order, int32_t* sorted_ids, int32_t* seg_of_pos, int64_t* uniq,
                   int32_t* seg_start, int64_t* inverse, int32_t* pair_seg, int32_t* n_uniq, int* err_flag) {
  using namespace smx;
  if (!idx || !order || !sorted_ids || !seg_of_pos || !uniq || !seg_start || !n_uniq || !workspace)
    return fail(SMX_ERR_ARG, "null pointer in plan build");
  if (n_pairs == 0 || n_pairs > 0x7fffffffull) return fail(SMX_ERR_SHAPE, "pair count %zu out of range", n_pairs);
  if (n_rows == 0 || n_rows > 0x100000000ull) return fail(SMX_ERR_SHAPE, "entity count %zu needs ids wider than 32 bits", n_rows);
  PlanScratch s;
  if (plan_scratch(n_pairs, n_rows, &s) != hipSuccess) return fail(SMX_ERR_HIP, "rocprim size query failed");
  if (workspace_bytes < s.total)
    return fail(SMX_ERR_WORKSPACE, "plan workspace too small: %zu < %zu", workspace_bytes, s.total);
  if (reinterpret_cast<uintptr_t>(workspace) & 255u) return fail(SMX_ERR_ARG, "workspace must be 256-byte aligned");
  hipStream_t st = as_stream(stream);
  char* ws = static_cast<char*>(workspace);
  unsigned* keys = reinterpret_cast<unsigned*>(ws + s.keys_off);
  unsigned* span_heads = reinterpret_cast<unsigned*>(ws + s.heads_off);
  unsigned* span_first = reinterpret_cast<unsigned*>(ws + s.first_off);
  void* temp = ws + s.temp_off;
  const int n = (int)n_pairs;
  const unsigned blocks = (unsigned)((n_pairs + 255) / 256);

  hipLaunchKernelGGL(plan_keys_kernel, dim3(blocks), dim3(256), 0, st, reinterpret_cast<const long long*>(idx), keys,
                     pair_seg, n, (unsigned long long)n_rows, err_flag);
  size_t tb = s.temp_bytes;
  hipError_t e = sort_pairs(temp, tb, keys, reinterpret_cast<unsigned*>(sorted_ids), order, n_pairs, key_bits(n_rows), st);
  if (e != hipSuccess) return fail(SMX_ERR_HIP, "radix sort: %s", hipGetErrorString(e));
  hipLaunchKernelGGL(plan_count_kernel, dim3((unsigned)s.spans), dim3(256), 0, st, sorted_ids, n, span_heads);
  hipLaunchKernelGGL(plan_offsets_kernel, dim3(1), dim3(1024), 0, st, span_heads, span_first, s.spans, n_uniq, seg_start,
                     n);
  hipLaunchKernelGGL(plan_emit_kernel, dim3((unsigned)s.spans), dim3(256), 0, st, sorted_ids, order, span_first,
                     seg_of_pos, reinterpret_cast<long long*>(uniq), seg_start, reinterpret_cast<long long*>(inverse),
                     pair_seg, n);
  return check_launch("plan build");
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
