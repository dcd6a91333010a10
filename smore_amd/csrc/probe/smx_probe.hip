// Bandwidth probes: what this GPU sustains for the access shapes the path is made of, measured with
// kernels that do nothing else.  bench.py reports the figures next to the step's achieved rate, so the
// fraction of the 8 TB/s nominal peak can be read against what a plain kernel reaches on the same box.
// Every probe keeps eight 16-byte loads (or stores) per lane in flight on a persistent grid.
// Built into a library of its own (libsmx_probe.so): measurement only, not part of the drop-in ABI.
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "../../../include/smx_probe.h"

namespace smx {

static thread_local char g_probe_err[256] = "";
static int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_probe_err, sizeof(g_probe_err), fmt, ap);
  va_end(ap);
  return code;
}
static int check_launch(const char* what) {
  const hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : fail(4, "%s: %s", what, hipGetErrorString(e));
}
static hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }
static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
constexpr int SMX_ERR_KIND = 1, SMX_ERR_SHAPE = 2, SMX_ERR_ARG = 3;

typedef float probe_vec4 __attribute__((ext_vector_type(4)));
constexpr int kProbeUnroll = 8;

__device__ __forceinline__ unsigned probe_hash(unsigned x) {
  x ^= x >> 16;
  x *= 0x7feb352dU;
  x ^= x >> 15;
  x *= 0x846ca68bU;
  x ^= x >> 16;
  return x;
}

// KIND 0: stream a, non-temporal loads.  1: stream a, plain loads.  2: copy a -> b.  3: a = 2 a in place.
// 4: fill a.
template <int KIND>
__global__ __launch_bounds__(256) void probe_stream_kernel(probe_vec4* __restrict__ a, probe_vec4* __restrict__ b,
                                                           size_t n4, float* sink) {
  probe_vec4 acc = {0.f, 0.f, 0.f, 0.f};
  const size_t stride = (size_t)gridDim.x * 256 * kProbeUnroll;
  for (size_t i = (size_t)blockIdx.x * 256 * kProbeUnroll + threadIdx.x; i < n4; i += stride) {
    probe_vec4 v[kProbeUnroll];
    if (KIND != 4) {
#pragma unroll
      for (int u = 0; u < kProbeUnroll; ++u) {
        const size_t j = min(i + (size_t)u * 256, n4 - 1);
        v[u] = KIND == 1 ? a[j] : __builtin_nontemporal_load(a + j);
      }
    }
#pragma unroll
    for (int u = 0; u < kProbeUnroll; ++u) {
      const size_t j = i + (size_t)u * 256;
      if (KIND <= 1) {
        acc += v[u];
      } else if (j < n4) {
        const probe_vec4 o = KIND == 4 ? probe_vec4{1.f, 2.f, 3.f, 4.f} : (KIND == 3 ? v[u] * 2.0f : v[u]);
        __builtin_nontemporal_store(o, (KIND == 2 ? b : a) + j);
      }
    }
  }
  if (KIND <= 1 && acc.x + acc.y + acc.z + acc.w == 123.456f) *sink = acc.x;  // keeps the loads alive
}

// Rows of row_f4 16-byte columns (at most 64: one load per lane) read at pseudo-random row numbers,
// one row per wavefront load, eight rows in flight per wavefront.
template <bool NT>
__global__ __launch_bounds__(256) void probe_rows_kernel(const probe_vec4* __restrict__ a, unsigned n_rows, int row_f4,
                                                         unsigned n_reads, float* sink) {
  const int lane = threadIdx.x & 63;
  const unsigned n_waves = gridDim.x * 4u, wid = blockIdx.x * 4u + (threadIdx.x >> 6);
  const unsigned groups = n_reads / kProbeUnroll;
  const int c = min(lane, row_f4 - 1);
  probe_vec4 acc = {0.f, 0.f, 0.f, 0.f};
  for (unsigned g = wid; g < groups; g += n_waves) {
    probe_vec4 v[kProbeUnroll];
#pragma unroll
    for (int r = 0; r < kProbeUnroll; ++r) {
      const unsigned row = (unsigned)__builtin_amdgcn_readfirstlane((int)(probe_hash(g * kProbeUnroll + r) % n_rows));
      const probe_vec4* p = a + (size_t)row * row_f4 + c;
      v[r] = NT ? __builtin_nontemporal_load(p) : *p;
    }
#pragma unroll
    for (int r = 0; r < kProbeUnroll; ++r) acc += v[r];
  }
  if (acc.x + acc.y + acc.z + acc.w == 123.456f) *sink = acc.x;
}

}  // namespace smx

extern "C" {

const char* smx_probe_last_error(void) { return smx::g_probe_err; }

int smx_probe_bandwidth(int kind, void* stream, void* a, void* b, size_t bytes, size_t row_bytes, size_t n_reads,
                        float* sink) {
  using namespace smx;
  if (!a || !sink || bytes < 4096 || (bytes & 15u)) return fail(SMX_ERR_ARG, "probe needs a buffer of a multiple of 16 bytes");
  if (!aligned16(a) || (b && !aligned16(b))) return fail(SMX_ERR_ARG, "probe buffers must be 16-byte aligned");
  hipStream_t st = as_stream(stream);
  int dev = 0, cus = 256;
  if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  const dim3 grid((unsigned)cus * 8u), block(256);
  probe_vec4* pa = static_cast<probe_vec4*>(a);
  probe_vec4* pb = static_cast<probe_vec4*>(b);
  const size_t n4 = bytes / 16;
  switch (kind) {
    case SMX_PROBE_READ_NT: hipLaunchKernelGGL(probe_stream_kernel<0>, grid, block, 0, st, pa, pb, n4, sink); break;
    case SMX_PROBE_READ: hipLaunchKernelGGL(probe_stream_kernel<1>, grid, block, 0, st, pa, pb, n4, sink); break;
    case SMX_PROBE_COPY:
      if (!b) return fail(SMX_ERR_ARG, "the copy probe needs a destination");
      hipLaunchKernelGGL(probe_stream_kernel<2>, grid, block, 0, st, pa, pb, n4, sink);
      break;
    case SMX_PROBE_UPDATE: hipLaunchKernelGGL(probe_stream_kernel<3>, grid, block, 0, st, pa, pb, n4, sink); break;
    case SMX_PROBE_FILL: hipLaunchKernelGGL(probe_stream_kernel<4>, grid, block, 0, st, pa, pb, n4, sink); break;
    case SMX_PROBE_ROWS:
    case SMX_PROBE_ROWS_NT: {
      if (row_bytes == 0 || (row_bytes & 15u) || row_bytes > 1024 || bytes / row_bytes == 0 ||
          bytes / row_bytes > 0xffffffffull || n_reads == 0 || n_reads > 0xffffffffull)
        return fail(SMX_ERR_SHAPE, "row probe: rows of 16..1024 bytes (multiple of 16), at most 2^32-1 rows and reads");
      const unsigned n_rows = (unsigned)(bytes / row_bytes);
      if (kind == SMX_PROBE_ROWS)
        hipLaunchKernelGGL(probe_rows_kernel<false>, grid, block, 0, st, pa, n_rows, (int)(row_bytes / 16), (unsigned)n_reads, sink);
      else
        hipLaunchKernelGGL(probe_rows_kernel<true>, grid, block, 0, st, pa, n_rows, (int)(row_bytes / 16), (unsigned)n_reads, sink);
      break;
    }
    default: return fail(SMX_ERR_KIND, "unknown probe %d", kind);
  }
  return check_launch("bandwidth probe");
}

}  // extern "C"
