// allocator.cpp -- allocator::allocator() of the ROCm backend and the memory
// counters of mlx/memory.h, over the caching device allocator of the C ABI
// (CUDA counterpart: mlx/backend/cuda/allocator.cpp:142-301,384-430).
//
// A Buffer wraps a rocm::RocmBuffer: HBM plus, once the CPU has asked for the
// data, a pinned host mirror and the bookkeeping of which side is current
// (residency.h).  Kernels take rocm::gpu_ptr<T>(array, stream); the CPU's way
// in is Buffer::raw_ptr().
#include "mlx/allocator.h"
#include "mlx/memory.h"

#include "allocator.h"
#include "device.h"

namespace mlx::core {

namespace rocm {

class RocmAllocator : public allocator::Allocator {
 public:
  allocator::Buffer malloc(size_t size) override {
    return allocator::Buffer{new RocmBuffer(size)}; // throws when out of memory
  }

  void free(allocator::Buffer buffer) override {
    delete static_cast<RocmBuffer*>(buffer.ptr());
  }

  size_t size(allocator::Buffer buffer) const override {
    auto* rec = static_cast<const RocmBuffer*>(buffer.ptr());
    return rec ? rec->size() : 0;
  }
};

RocmAllocator& rocm_allocator() {
  static RocmAllocator* a = new RocmAllocator; // leaked: outlives static arrays
  return *a;
}

} // namespace rocm

namespace allocator {

Allocator& allocator() {
  return rocm::rocm_allocator();
}

void* Buffer::raw_ptr() {
  auto* rec = static_cast<rocm::RocmBuffer*>(ptr_);
  return rec ? rec->host_access() : nullptr;
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
