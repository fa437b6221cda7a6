// Error channel and version query of the C ABI.
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>

#include "common.hpp"

namespace arctic {

static thread_local char g_last_error[512] = "";

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
  return code;
}

// Turns a failed kernel launch into an error code (the reference uses
// C10_CUDA_KERNEL_LAUNCH_CHECK, csrc/custom_ops/speculator_ln.cu:233).
int check_launch(const char *what) {
  const hipError_t err = hipGetLastError();
  if (err == hipSuccess) return ARCTIC_OK;
  return fail(ARCTIC_ERR_LAUNCH, "%s: kernel launch failed: %s", what, hipGetErrorString(err));
}

}  // namespace arctic

extern "C" int arctic_abi_version(void) { return ARCTIC_ABI_VERSION; }

extern "C" const char *arctic_last_error(void) { return arctic::g_last_error; }
