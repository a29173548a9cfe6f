// runtime.hip -- device memory with explicit residency, streams and events.
//
// The allocator is what a ROCm build of MLX puts behind allocator::malloc/free
// (mlx/allocator.h:52-75) and the counters of mlx/memory.h.  Unlike the unified
// memory the other GPU backends assume, every buffer here is device-resident
// (hipMalloc); host access goes through explicit copies into pinned staging
// memory.  Freed buffers are kept in a size-bucketed cache (the size classes of
// mlx/backend/cuda/allocator.cpp:22-29: tiny -> 8 B, small -> next power of two,
// large -> whole 16 KiB pages) and handed back on the next request of the same
// class; the cache is trimmed, least recently freed buffer first, above the cache
// limit, when active + cached + requested bytes would pass the memory limit
// (95 % of the device's memory unless set; the relief valve of
// mlx/backend/cuda/allocator.cpp:186-191), and emptied when hipMalloc runs out of
// memory.  A request larger than the device's memory fails without reaching HIP.
#include <map>
#include <mutex>
#include <unordered_map>

#include "common.h"

namespace mlxrocm {

namespace {

constexpr size_t kSmall = 8;
constexpr size_t kPage = 16384;

size_t size_class(size_t size) {
  if (size <= kSmall) {
    return kSmall;
  }
  if (size < kPage) {
    size_t p = 16;
    while (p < size) {
      p <<= 1;
    }
    return p;
  }
  return (size + kPage - 1) / kPage * kPage;
}

class DeviceAllocator {
 public:
  int malloc(void** out, size_t size) {
    if (out == nullptr) {
      return fail(MLXROCM_INVALID_ARGUMENT, "[malloc] null result pointer");
    }
    *out = nullptr;
    if (size == 0) {
      return MLXROCM_OK; // MLX hands out an empty Buffer for size 0
    }
    const size_t cls = size_class(size);
    std::lock_guard<std::mutex> lock(mu_);
    // Reuse: the smallest cached buffer of at least this class, if it would
    // not waste more than half of itself.
    auto it = cache_.lower_bound(cls);
    if (it != cache_.end() && it->first <= cls * 2) {
      void* p = it->second.ptr;
      const size_t got = it->first;
      lru_.erase(it->second.seq);
      cache_.erase(it);
      cached_bytes_ -= got;
      live_[p] = got;
      note_active(got);
      *out = p;
      return MLXROCM_OK;
    }
    ask_device();
    if (cls < size || cls > total_memory_) {
      return fail(
          MLXROCM_OUT_OF_MEMORY,
          "[malloc] unable to allocate %zu bytes: the device holds %zu",
          size,
          total_memory_);
    }
    // memory pressure: give cached buffers back before asking for more
    if (cached_bytes_ > 0) {
      const size_t want = active_bytes_ + cached_bytes_ + cls;
      if (want > memory_limit_) {
        const size_t over = want - memory_limit_;
        release_cache(over >= cached_bytes_ ? 0 : cached_bytes_ - over);
      }
    }
    void* p = nullptr;
    hipError_t err = hipMalloc(&p, cls);
    if (err == hipErrorOutOfMemory) {
      (void)hipGetLastError();
      release_cache(0);
      err = hipMalloc(&p, cls);
    }
    if (err != hipSuccess) {
      (void)hipGetLastError();
      return fail(
          err == hipErrorOutOfMemory ? MLXROCM_OUT_OF_MEMORY : MLXROCM_HIP_ERROR,
          "[malloc] unable to allocate %zu bytes: %s",
          size,
          hipGetErrorString(err));
    }
    live_[p] = cls;
    note_active(cls);
    *out = p;
    return MLXROCM_OK;
  }

  int free(void* p) {
    if (p == nullptr) {
      return MLXROCM_OK;
    }
    std::lock_guard<std::mutex> lock(mu_);
    auto it = live_.find(p);
    if (it == live_.end()) {
      return fail(
          MLXROCM_INVALID_ARGUMENT, "[free] pointer %p is not a live buffer", p);
    }
    const size_t sz = it->second;
    live_.erase(it);
    active_bytes_ -= sz;
    const uint64_t seq = next_seq_++;
    lru_[seq] = cache_.emplace(sz, Cached{p, seq});
    cached_bytes_ += sz;
    if (cached_bytes_ > cache_limit_) {
      release_cache(cache_limit_);
    }
    return MLXROCM_OK;
  }

  size_t buffer_size(const void* p) {
    std::lock_guard<std::mutex> lock(mu_);
    auto it = live_.find(const_cast<void*>(p));
    return it == live_.end() ? 0 : it->second;
  }

  size_t active() {
    std::lock_guard<std::mutex> lock(mu_);
    return active_bytes_;
  }
  size_t peak() {
    std::lock_guard<std::mutex> lock(mu_);
    return peak_bytes_;
  }
  void reset_peak() {
    std::lock_guard<std::mutex> lock(mu_);
    peak_bytes_ = 0;
  }
  size_t cached() {
    std::lock_guard<std::mutex> lock(mu_);
    return cached_bytes_;
  }
  size_t set_cache_limit(size_t limit) {
    std::lock_guard<std::mutex> lock(mu_);
    const size_t prev = cache_limit_;
    cache_limit_ = limit;
    if (cached_bytes_ > cache_limit_) {
      release_cache(cache_limit_);
    }
    return prev;
  }
  size_t set_memory_limit(size_t limit) {
    std::lock_guard<std::mutex> lock(mu_);
    ask_device();
    const size_t prev = memory_limit_;
    memory_limit_ = limit;
    return prev;
  }
  size_t memory_limit() {
    std::lock_guard<std::mutex> lock(mu_);
    ask_device();
    return memory_limit_;
  }
  void clear_cache() {
    std::lock_guard<std::mutex> lock(mu_);
    release_cache(0);
  }

 private:
  // The device's memory size and, unless a limit has been set, the default
  // limit derived from it; asked once, on first use.
  void ask_device() {
    if (total_memory_ != 0) {
      return;
    }
    size_t free_now = 0;
    if (hipMemGetInfo(&free_now, &total_memory_) != hipSuccess || total_memory_ == 0) {
      (void)hipGetLastError();
      total_memory_ = static_cast<size_t>(-1);
      return;
    }
    if (memory_limit_ == static_cast<size_t>(-1)) {
      memory_limit_ = total_memory_ / 100 * 95;
    }
  }

  void note_active(size_t sz) {
    active_bytes_ += sz;
    if (active_bytes_ > peak_bytes_) {
      peak_bytes_ = active_bytes_;
    }
  }

  // Frees cached buffers, least recently freed first, until at most `target`
  // bytes remain.
  void release_cache(size_t target) {
    while (cached_bytes_ > target && !lru_.empty()) {
      auto oldest = lru_.begin();
      auto it = oldest->second;
      (void)hipFree(it->second.ptr);
      cached_bytes_ -= it->first;
      cache_.erase(it);
      lru_.erase(oldest);
    }
  }

  struct Cached {
    void* ptr;
    uint64_t seq;
  };
  using Cache = std::multimap<size_t, Cached>;

  std::mutex mu_;
  std::unordered_map<void*, size_t> live_;
  Cache cache_; // by size class
  std::map<uint64_t, Cache::iterator> lru_; // by time of the free
  uint64_t next_seq_ = 0;
  size_t total_memory_ = 0; // 0: not asked yet
  size_t active_bytes_ = 0;
  size_t peak_bytes_ = 0;
  size_t cached_bytes_ = 0;
  size_t cache_limit_ = static_cast<size_t>(-1);
  size_t memory_limit_ = static_cast<size_t>(-1);
};

DeviceAllocator& allocator() {
  // Leaked on purpose: buffers may be freed from static destructors of the
  // host program after this translation unit's statics are gone.
  static DeviceAllocator* a = new DeviceAllocator();
  return *a;
}

} // namespace

} // namespace mlxrocm

using namespace mlxrocm;

extern "C" int mlxrocm_malloc(void** ptr, size_t size) {
  return allocator().malloc(ptr, size);
}
extern "C" int mlxrocm_free(void* ptr) {
  return allocator().free(ptr);
}
extern "C" size_t mlxrocm_buffer_size(const void* ptr) {
  return allocator().buffer_size(ptr);
}
extern "C" size_t mlxrocm_get_active_memory(void) {
  return allocator().active();
}
extern "C" size_t mlxrocm_get_peak_memory(void) {
  return allocator().peak();
}
extern "C" void mlxrocm_reset_peak_memory(void) {
  allocator().reset_peak();
}
extern "C" size_t mlxrocm_get_cache_memory(void) {
  return allocator().cached();
}
extern "C" size_t mlxrocm_set_cache_limit(size_t limit) {
  return allocator().set_cache_limit(limit);
}
extern "C" size_t mlxrocm_set_memory_limit(size_t limit) {
  return allocator().set_memory_limit(limit);
}
extern "C" size_t mlxrocm_get_memory_limit(void) {
  return allocator().memory_limit();
}
extern "C" void mlxrocm_clear_cache(void) {
  allocator().clear_cache();
}

extern "C" int mlxrocm_host_malloc(void** ptr, size_t size) {
  if (ptr == nullptr) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[host_malloc] null result pointer");
  }
  *ptr = nullptr;
  if (size == 0) {
    return MLXROCM_OK;
  }
  MLXROCM_HIP_TRY(hipHostMalloc(ptr, size, hipHostMallocDefault));
  return MLXROCM_OK;
}
extern "C" int mlxrocm_host_free(void* ptr) {
  if (ptr != nullptr) {
    MLXROCM_HIP_TRY(hipHostFree(ptr));
  }
  return MLXROCM_OK;
}

extern "C" int
mlxrocm_memcpy_h2d(void* dst, const void* src, size_t n, mlxrocm_stream_t s) {
  if (n == 0) {
    return MLXROCM_OK;
  }
  MLXROCM_HIP_TRY(hipMemcpyAsync(
      dst, src, n, hipMemcpyHostToDevice, static_cast<hipStream_t>(s)));
  return MLXROCM_OK;
}
extern "C" int
mlxrocm_memcpy_d2h(void* dst, const void* src, size_t n, mlxrocm_stream_t s) {
  if (n == 0) {
    return MLXROCM_OK;
  }
  MLXROCM_HIP_TRY(hipMemcpyAsync(
      dst, src, n, hipMemcpyDeviceToHost, static_cast<hipStream_t>(s)));
  return MLXROCM_OK;
}
extern "C" int
mlxrocm_memcpy_d2d(void* dst, const void* src, size_t n, mlxrocm_stream_t s) {
  if (n == 0) {
    return MLXROCM_OK;
  }
  MLXROCM_HIP_TRY(hipMemcpyAsync(
      dst, src, n, hipMemcpyDeviceToDevice, static_cast<hipStream_t>(s)));
  return MLXROCM_OK;
}

extern "C" int mlxrocm_stream_create(mlxrocm_stream_t* stream) {
  if (stream == nullptr) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[stream_create] null result pointer");
  }
  hipStream_t s = nullptr;
  // Default priority only: mixed-priority streams are not used anywhere.
  MLXROCM_HIP_TRY(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
  *stream = s;
  return MLXROCM_OK;
}
extern "C" int mlxrocm_stream_destroy(mlxrocm_stream_t stream) {
  if (stream != nullptr) {
    MLXROCM_HIP_TRY(hipStreamDestroy(static_cast<hipStream_t>(stream)));
  }
  return MLXROCM_OK;
}
extern "C" int mlxrocm_stream_synchronize(mlxrocm_stream_t stream) {
  MLXROCM_HIP_TRY(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
  return MLXROCM_OK;
}

extern "C" int mlxrocm_event_create(mlxrocm_event_t* event) {
  if (event == nullptr) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[event_create] null result pointer");
  }
  hipEvent_t e = nullptr;
  MLXROCM_HIP_TRY(hipEventCreate(&e));
  *event = e;
  return MLXROCM_OK;
}
extern "C" int mlxrocm_event_create_blocking(mlxrocm_event_t* event) {
  if (event == nullptr) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[event_create] null result pointer");
  }
  hipEvent_t e = nullptr;
  MLXROCM_HIP_TRY(hipEventCreateWithFlags(&e, hipEventBlockingSync | hipEventDisableTiming));
  *event = e;
  return MLXROCM_OK;
}
extern "C" int mlxrocm_event_destroy(mlxrocm_event_t event) {
  if (event != nullptr) {
    MLXROCM_HIP_TRY(hipEventDestroy(static_cast<hipEvent_t>(event)));
  }
  return MLXROCM_OK;
}
extern "C" int mlxrocm_event_record(mlxrocm_event_t event, mlxrocm_stream_t stream) {
  MLXROCM_HIP_TRY(hipEventRecord(
      static_cast<hipEvent_t>(event), static_cast<hipStream_t>(stream)));
  return MLXROCM_OK;
}
extern "C" int mlxrocm_event_wait(mlxrocm_event_t event, mlxrocm_stream_t stream) {
  MLXROCM_HIP_TRY(hipStreamWaitEvent(
      static_cast<hipStream_t>(stream), static_cast<hipEvent_t>(event), 0));
  return MLXROCM_OK;
}
extern "C" int mlxrocm_event_synchronize(mlxrocm_event_t event) {
  MLXROCM_HIP_TRY(hipEventSynchronize(static_cast<hipEvent_t>(event)));
  return MLXROCM_OK;
}
extern "C" int mlxrocm_event_query(mlxrocm_event_t event) {
  hipError_t err = hipEventQuery(static_cast<hipEvent_t>(event));
  if (err == hipSuccess) {
    return 1;
  }
  if (err == hipErrorNotReady) {
    (void)hipGetLastError();
    return 0;
  }
  return hip_fail(err, "hipEventQuery");
}
extern "C" int mlxrocm_event_elapsed_ms(
    float* ms,
    mlxrocm_event_t start,
    mlxrocm_event_t stop) {
  if (ms == nullptr) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[event_elapsed_ms] null result pointer");
  }
  MLXROCM_HIP_TRY(hipEventElapsedTime(
      ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)));
  return MLXROCM_OK;
}

extern "C" int mlxrocm_device_count(void) {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  return n;
}

extern "C" int mlxrocm_device_info(
    int device,
    char* name,
    int* compute_units,
    size_t* total_memory,
    int* clock_khz) {
  hipDeviceProp_t prop;
  MLXROCM_HIP_TRY(hipGetDeviceProperties(&prop, device));
  if (name != nullptr) {
    snprintf(name, 256, "%s (%s)", prop.name, prop.gcnArchName);
  }
  if (compute_units != nullptr) {
    *compute_units = prop.multiProcessorCount;
  }
  if (total_memory != nullptr) {
    *total_memory = prop.totalGlobalMem;
  }
  if (clock_khz != nullptr) {
    *clock_khz = prop.clockRate;
  }
  return MLXROCM_OK;
}
