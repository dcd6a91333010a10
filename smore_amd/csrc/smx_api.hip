// Version, error text and name lookup of the C ABI.
#include <atomic>
#include <cstring>

#include "smx_common.h"
#include "smx_functors.h"

namespace smx {

static thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(SMX_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
  return SMX_OK;
}

static std::atomic<int> g_serial_backward{0};
bool serial_backward() { return g_serial_backward.load(std::memory_order_relaxed) != 0; }

}  // namespace smx

extern "C" {

int smx_version(void) { return 2; }

int smx_set_option(int option, int value) {
  if (option == SMX_OPTION_SERIAL_BACKWARD) {
    smx::g_serial_backward.store(value ? 1 : 0, std::memory_order_relaxed);
    return SMX_OK;
  }
  return smx::fail(SMX_ERR_ARG, "unknown option %d", option);
}

const char* smx_last_error(void) { return smx::g_err; }

int smx_kind_from_name(const char* name) {
  static const char* const names[smx::kNumKinds] = {
      "l1", "l2", "box_out", "box_in", "rotate", "beta_kl", "complex", "distmult", "beta_l2", "beta_fisher_approx"};
  if (!name) return -1;
  for (int k = 0; k < smx::kNumKinds; ++k)
    if (std::strcmp(name, names[k]) == 0) return k;
  return -1;
}

}  // extern "C"
