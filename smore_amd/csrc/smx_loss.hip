// The sample loss that sits between the scoring forward and its backward, and its gradient.
//
// Replaces the dozen element-wise / row-reduction tensor passes of
// smore/training/train_process.py:194-213 over the [B,K] negative logits:
//   x = neg * is_negative_mat;  s_b = sum_k softmax(x T)_k.detach() logsigmoid(-x_k)  | mean_k logsigmoid(-x_k)
//   p_b = logsigmoid(pos_b);    loss = (-sum W_b p_b - sum W_b s_b) / 2 / world_size,  W_b = w_b / sum w | 1/B
// with one pass that also writes d loss / d logit, i.e. the upstream gradient the scoring backward
// consumes -- autograd is not needed between the two.  One workgroup per query; every reduction has
// a fixed order (DPP inside a wavefront, wavefront order across the workgroup, query order at the end).
#include <cmath>
#include <mutex>

#include "smx_common.h"
#include "smx_wave.h"

namespace smx {

struct LossArgs {
  const float* pos;     // [B]
  const float* neg;     // [B,K]
  const float* mask;    // [B,K] or null
  const float* weight;  // [B] or null
  int B, K;
  float temperature;    // > 0: self-adversarial weights, 0: plain mean over K
  float scale;
  float* wsum;          // device scalar: sum of weights (or B)
  float* per_query;     // [B,2]: W_b logsigmoid(pos_b), W_b s_b
  float* out_loss;      // [2]
  float* gpos;          // [B]
  float* gneg;          // [B,K]
};

// Sum / max over the workgroup (256 threads), same value in every thread, fixed order.
__device__ __forceinline__ float block_sum(float v, float* lds) {
  v = wave_sum_f32(v);
  __syncthreads();  // lds may still be read from the previous reduction
  if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = v;
  __syncthreads();
  return ((lds[0] + lds[1]) + lds[2]) + lds[3];
}
__device__ __forceinline__ float block_max(float v, float* lds) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off));
  __syncthreads();
  if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = v;
  __syncthreads();
  return fmaxf(fmaxf(lds[0], lds[1]), fmaxf(lds[2], lds[3]));
}

__device__ __forceinline__ float log_sigmoid(float x) { return fminf(x, 0.f) - log1pf(expf(-fabsf(x))); }
__device__ __forceinline__ float sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }

__global__ __launch_bounds__(256) void loss_weight_sum_kernel(LossArgs A) {
  __shared__ float lds[4];
  float part = 0.f;
  for (int b = threadIdx.x; b < A.B; b += 256) part += A.weight[b];
  const float total = block_sum(part, lds);
  if (threadIdx.x == 0) *A.wsum = total;
}

__global__ __launch_bounds__(256) void loss_rows_kernel(LossArgs A) {
  __shared__ float lds[4];
  const int b = blockIdx.x;
  const float* __restrict__ neg = A.neg + (size_t)b * A.K;
  const float* __restrict__ mask = A.mask ? A.mask + (size_t)b * A.K : nullptr;
  float* __restrict__ gneg = A.gneg + (size_t)b * A.K;
  const float W = A.weight ? A.weight[b] / *A.wsum : 1.0f / (float)A.B;
  const float T = A.temperature;

  float mx = 0.f, inv_z = 1.0f / (float)A.K;
  if (T > 0.f) {
    float m = -INFINITY;
    for (int k = threadIdx.x; k < A.K; k += 256) m = fmaxf(m, neg[k] * (mask ? mask[k] : 1.f) * T);
    mx = block_max(m, lds);
    float z = 0.f;
    for (int k = threadIdx.x; k < A.K; k += 256) z += expf(neg[k] * (mask ? mask[k] : 1.f) * T - mx);
    inv_z = 1.0f / block_sum(z, lds);
  }
  float s = 0.f;
  for (int k = threadIdx.x; k < A.K; k += 256) {
    const float mk = mask ? mask[k] : 1.f;
    const float x = neg[k] * mk;
    const float a = T > 0.f ? expf(x * T - mx) * inv_z : inv_z;
    s += a * log_sigmoid(-x);
    gneg[k] = A.scale * W * a * sigmoid(x) * mk;
  }
  s = block_sum(s, lds);
  if (threadIdx.x == 0) {
    const float p = A.pos[b];
    A.per_query[2 * b] = W * log_sigmoid(p);
    A.per_query[2 * b + 1] = W * s;
    A.gpos[b] = -A.scale * W * sigmoid(-p);
  }
}

__global__ __launch_bounds__(256) void loss_finish_kernel(LossArgs A) {
  __shared__ float lds[4];
  float p = 0.f, s = 0.f;
  for (int b = threadIdx.x; b < A.B; b += 256) {
    p += A.per_query[2 * b];
    s += A.per_query[2 * b + 1];
  }
  p = block_sum(p, lds);
  s = block_sum(s, lds);
  if (threadIdx.x == 0) {
    A.out_loss[0] = -p;
    A.out_loss[1] = -s;
  }
}

static size_t loss_ws_bytes(size_t B) { return ((2 * B + 1) * sizeof(float) + 255) & ~(size_t)255; }

// Scratch of smx_sample_loss_static: the per-query partial losses and the weight sum that smx_sample_loss
// keeps in the caller's workspace.  One copy per device, held until the process ends.
constexpr size_t kStaticLossMaxB = SMX_SAMPLE_LOSS_STATIC_MAX_QUERIES;
static __device__ __align__(256) float scratch[2 * kStaticLossMaxB + 64];

// The array's name is a host-side stand-in: its device address is asked for once per device, with that
// device current, and kept.
static float* static_scratch() {
  static std::mutex mu;
  static float* per_device[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return nullptr;
  std::lock_guard<std::mutex> lock(mu);
  if (!per_device[dev]) {
    float* ptr = nullptr;
    if (hipGetSymbolAddress(reinterpret_cast<void**>(&ptr), HIP_SYMBOL(scratch)) != hipSuccess) return nullptr;
    per_device[dev] = ptr;
  }
  return per_device[dev];
}

// Argument checks and launches shared by the two entry points; `buf` holds 2 B + 1 floats.
static int launch_loss(void* stream, const float* pos, const float* neg, const float* mask, const float* weight,
                       size_t B, size_t K, double temperature, double scale, float* out_loss, float* gpos, float* gneg,
                       float* buf) {
  if (!pos || !neg || !out_loss || !gpos || !gneg || !buf) return fail(SMX_ERR_ARG, "null pointer in sample loss");
  if (B == 0 || K == 0 || B > 0x7fffffffull || K > 0x7fffffffull) return fail(SMX_ERR_SHAPE, "empty or oversized batch");
  if (!(temperature >= 0.0)) return fail(SMX_ERR_ARG, "adversarial temperature must be >= 0 (0 = plain mean)");
  LossArgs A{};
  A.pos = pos;
  A.neg = neg;
  A.mask = mask;
  A.weight = weight;
  A.B = (int)B;
  A.K = (int)K;
  A.temperature = (float)temperature;
  A.scale = (float)scale;
  A.per_query = buf;
  A.wsum = buf + 2 * B;
  A.out_loss = out_loss;
  A.gpos = gpos;
  A.gneg = gneg;
  hipStream_t st = as_stream(stream);
  if (weight) hipLaunchKernelGGL(loss_weight_sum_kernel, dim3(1), dim3(256), 0, st, A);
  hipLaunchKernelGGL(loss_rows_kernel, dim3((unsigned)B), dim3(256), 0, st, A);
  hipLaunchKernelGGL(loss_finish_kernel, dim3(1), dim3(256), 0, st, A);
  return check_launch("sample loss");
}

}  // namespace smx

extern "C" {

size_t smx_sample_loss_workspace_bytes(size_t B) { return smx::loss_ws_bytes(B); }

int smx_sample_loss(void* stream, const float* pos, const float* neg, const float* mask, const float* weight,
                    size_t B, size_t K, double temperature, double scale, float* out_loss, float* gpos, float* gneg,
                    void* workspace, size_t workspace_bytes) {
  using namespace smx;
  if (!workspace) return fail(SMX_ERR_ARG, "null pointer in sample loss");
  if (workspace_bytes < loss_ws_bytes(B))
    return fail(SMX_ERR_WORKSPACE, "loss workspace too small: %zu < %zu", workspace_bytes, loss_ws_bytes(B));
  return launch_loss(stream, pos, neg, mask, weight, B, K, temperature, scale, out_loss, gpos, gneg,
                     static_cast<float*>(workspace));
}

int smx_sample_loss_static(void* stream, const float* pos, const float* neg, const float* mask, const float* weight,
                           size_t B, size_t K, double temperature, double scale, float* out_loss, float* gpos,
                           float* gneg) {
  using namespace smx;
  if (B > kStaticLossMaxB)
    return fail(SMX_ERR_SHAPE, "smx_sample_loss_static takes at most %zu queries per call, got %zu", kStaticLossMaxB, B);
  float* buf = static_scratch();
  if (!buf) return fail(SMX_ERR_HIP, "cannot get the device address of the library's scratch array");
  // every float of the scratch this call reads (2 B partial losses, the weight sum when weights are given)
  // is written by its own kernels first: nothing has to start at zero
  return launch_loss(stream, pos, neg, mask, weight, B, K, temperature, scale, out_loss, gpos, gneg, buf);
}

}  // extern "C"
