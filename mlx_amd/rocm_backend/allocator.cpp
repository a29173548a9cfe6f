// allocator.cpp -- allocator::allocator() of the ROCm backend: device-resident
// buffers with explicit host residency.
//
// MLX's other GPU backends hand out memory the CPU can touch directly (unified
// memory on Metal, managed memory on CUDA, mlx/backend/cuda/allocator.cpp:252-301).
// Here a Buffer wraps a small record {device pointer, size, pinned host mirror}.
// Kernels use the device pointer (rocm::gpu_ptr<T>(array, stream));
// Buffer::raw_ptr() -- the CPU's way in -- makes
// the data host-visible on demand: it synchronizes, copies device -> pinned
// host and returns the mirror, which gpu_ptr() uploads again before the next kernel
// that touches the buffer.  The CUDA backend does the same movement implicitly
// through managed-memory migration (mlx/backend/cuda/allocator.cpp:252-301).
#include <mutex>
#include <stdexcept>
#include <unordered_set>

#include "mlx/allocator.h"
#include "mlx/memory.h"

#include "allocator.h"
#include "device.h"

namespace mlx::core {

namespace rocm {

class RocmAllocator : public allocator::Allocator {
 public:
  allocator::Buffer malloc(size_t size) override {
    auto* rec = new RocmBuffer;
    rec->size = size;
    int rc = mlxrocm_malloc(&rec->device, size);
    if (rc != MLXROCM_OK) {
      delete rec;
      check(rc);
    }
    return allocator::Buffer{rec};
  }

  void free(allocator::Buffer buffer) override {
    auto* rec = static_cast<RocmBuffer*>(buffer.ptr());
    if (rec == nullptr) {
      return;
    }
    (void)mlxrocm_free(rec->device);
    (void)mlxrocm_host_free(rec->host);
    delete rec;
  }

  size_t size(allocator::Buffer buffer) const override {
    auto* rec = static_cast<const RocmBuffer*>(buffer.ptr());
    return rec ? rec->size : 0;
  }
};

RocmAllocator& rocm_allocator() {
  static RocmAllocator* a = new RocmAllocator; // leaked: outlives static arrays
  return *a;
}

// Device pointer of a buffer, writing a dirty host mirror back first.
void* device_ptr(allocator::Buffer buffer, mlxrocm_stream_t stream) {
  auto* rec = static_cast<RocmBuffer*>(buffer.ptr());
  if (rec == nullptr) {
    return nullptr;
  }
  if (rec->host_dirty) {
    check(mlxrocm_memcpy_h2d(rec->device, rec->host, rec->size, stream));
    rec->host_dirty = false;
  }
  return rec->device;
}

} // namespace rocm

namespace allocator {

Allocator& allocator() {
  return rocm::rocm_allocator();
}

void* Buffer::raw_ptr() {
  auto* rec = static_cast<rocm::RocmBuffer*>(ptr_);
  if (rec == nullptr) {
    return nullptr;
  }
  if (rec->host == nullptr) {
    rocm::check(mlxrocm_host_malloc(&rec->host, rec->size));
  }
  // Explicit residency: bring the device contents to the host mirror.
  rocm::check(mlxrocm_memcpy_d2h(rec->host, rec->device, rec->size, nullptr));
  rocm::check(mlxrocm_stream_synchronize(nullptr));
  rec->host_dirty = true; // the caller may write through the pointer
  return rec->host;
}

} // namespace allocator

size_t get_active_memory() {
  return mlxrocm_get_active_memory();
}
size_t get_peak_memory() {
  return mlxrocm_get_peak_memory();
}
void reset_peak_memory() {
  mlxrocm_reset_peak_memory();
}
size_t get_cache_memory() {
  return mlxrocm_get_cache_memory();
}
size_t set_memory_limit(size_t limit) {
  return mlxrocm_set_memory_limit(limit);
}
size_t get_memory_limit() {
  return mlxrocm_get_memory_limit();
}
size_t set_cache_limit(size_t limit) {
  return mlxrocm_set_cache_limit(limit);
}
void clear_cache() {
  mlxrocm_clear_cache();
}

} // namespace mlx::core
