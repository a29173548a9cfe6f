// errors.hip -- thread-local error slot of the C ABI.
#include <cstdarg>
#include <cstdio>

#include "common.h"

namespace mlxrocm {

namespace {
thread_local char g_last_error[512] = "";
}

int fail(int status, const char* fmt, ...) {
  va_list args;
  va_start(args, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, args);
  va_end(args);
  return status;
}

int hip_fail(hipError_t err, const char* what) {
  snprintf(
      g_last_error,
      sizeof(g_last_error),
      "HIP error %d (%s) in %s",
      static_cast<int>(err),
      hipGetErrorString(err),
      what);
  return err == hipErrorOutOfMemory ? MLXROCM_OUT_OF_MEMORY : MLXROCM_HIP_ERROR;
}

} // namespace mlxrocm

extern "C" int mlxrocm_abi_version(void) {
  return MLXROCM_ABI_VERSION;
}

extern "C" const char* mlxrocm_last_error(void) {
  return mlxrocm::g_last_error;
}
