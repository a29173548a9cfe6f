// errors.hip -- thread-local error slot of the C ABI and the roctx ranges of
// its entry points.
#include <dlfcn.h>

#include <cstdarg>
#include <cstdio>
#include <mutex>

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

namespace {

struct Markers {
  int (*push)(const char*) = nullptr;
  int (*pop)() = nullptr;
};

const Markers& markers() {
  static Markers m;
  static std::once_flag once;
  std::call_once(once, [] {
    // rocprofv3's marker library; older tools ship the same two symbols in
    // libroctx64.
    for (const char* name : {"librocprofiler-sdk-roctx.so.1", "librocprofiler-sdk-roctx.so",
                             "libroctx64.so.4", "libroctx64.so"}) {
      if (void* lib = dlopen(name, RTLD_NOW | RTLD_LOCAL)) {
        auto push = reinterpret_cast<int (*)(const char*)>(dlsym(lib, "roctxRangePushA"));
        auto pop = reinterpret_cast<int (*)()>(dlsym(lib, "roctxRangePop"));
        if (push != nullptr && pop != nullptr) {
          m.push = push;
          m.pop = pop;
          return;
        }
      }
    }
  });
  return m;
}

} // namespace

ApiRange::ApiRange(const char* name) : open_(false) {
  const Markers& m = markers();
  if (m.push != nullptr) {
    m.push(name);
    open_ = true;
  }
}

ApiRange::~ApiRange() {
  if (open_) {
    markers().pop();
  }
}

} // namespace mlxrocm

extern "C" int mlxrocm_abi_version(void) {
  return MLXROCM_ABI_VERSION;
}

extern "C" const char* mlxrocm_last_error(void) {
  return mlxrocm::g_last_error;
}
