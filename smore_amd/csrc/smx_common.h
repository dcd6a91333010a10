// Host-side helpers shared by the translation units of libsmore_amd.so.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstddef>
#include <cstdint>
#include <cstdio>

#include "../../include/smore_amd.h"

namespace smx {

constexpr int kWave = 64;  // gfx950 wavefront

// Records the message returned by smx_last_error() and hands back `code`.
int fail(int code, const char* fmt, ...);

// Checks the launch that just happened on this thread.
int check_launch(const char* what);

// smx_set_option(SMX_OPTION_SERIAL_BACKWARD, ..): the backward keeps to the caller's stream
bool serial_backward();

constexpr int kMaxSources = 4;  // index streams one entity pass can reduce together (SMX_MAX_PAIR_SOURCES)

// Several index streams behind one segment plan: source i holds pairs [B * (K_0 + .. + K_i-1), + B * K_i) of the
// plan, with its own score / upstream gradient / sign-code arrays; all sources share the query tensors.
struct PairSources {
  int n;
  const float* score[kMaxSources];
  const float* gscore[kMaxSources];
  const unsigned char* codes[kMaxSources];
  size_t K[kMaxSources];
  size_t B[kMaxSources];        // queries of the source, and the row of q1 / q2 (group of U rows) where they start
  size_t q_first[kMaxSources];
  // union queries: U branch rows per query in q1 / q2, and per source the branch that gave each pair's logit
  // (null when U == 1)
  const unsigned char* winner[kMaxSources];
  size_t U;
  // behind the pairs of all sources the plan may hold n_grad more entries whose gradient autograd has already
  // materialised as a row each (plain lookups of the step: anchor entities): grad_rows[n_grad, row]
  const float* grad_rows;
  size_t n_grad;
};

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace smx
