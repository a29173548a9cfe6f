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

namespace {
struct Rehearsal {
  char* buf = nullptr;
  size_t cap = 0;
  size_t len = 0;
  bool active = false;
};
thread_local Rehearsal g_rehearsal;
} // namespace

RehearsalScope::RehearsalScope(char* buf, size_t cap) {
  g_rehearsal.buf = buf;
  g_rehearsal.cap = cap;
  g_rehearsal.len = 0;
  g_rehearsal.active = true;
  if (buf != nullptr && cap > 0) {
    buf[0] = '\0';
  }
}

RehearsalScope::~RehearsalScope() {
  g_rehearsal = Rehearsal{};
}

bool rehearsing() {
  return g_rehearsal.active;
}

int note_launch(const char* fmt, ...) {
  Rehearsal& r = g_rehearsal;
  if (!r.active || r.buf == nullptr || r.len + 2 >= r.cap) {
    return MLXROCM_OK;
  }
  if (r.len > 0) {
    r.buf[r.len++] = '+';
  }
  va_list args;
  va_start(args, fmt);
  const int n = vsnprintf(r.buf + r.len, r.cap - r.len, fmt, args);
  va_end(args);
  if (n > 0) {
    const size_t room = r.cap - r.len - 1;
    r.len += static_cast<size_t>(n) < room ? static_cast<size_t>(n) : room;
  }
  r.buf[r.len] = '\0';
  return MLXROCM_OK;
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
