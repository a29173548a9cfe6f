// allocator.h -- the device-pointer accessor eval_gpu bodies use (the
// counterpart of gpu_ptr<T>, mlx/backend/cuda/utils.h:26-39).  An
// allocator::Buffer of this backend points at a rocm::RocmBuffer (residency.h).
#pragma once

#include <type_traits>

#include "mlx/array.h"

#include "residency.h"

namespace mlx::core::rocm {

// Device address of a buffer for kernels on `stream`; uploads the host mirror
// first when the CPU touched the buffer last.
inline void* device_ptr(allocator::Buffer buffer, mlxrocm_stream_t stream, bool will_write) {
  auto* rec = static_cast<RocmBuffer*>(buffer.ptr());
  return rec ? rec->device_access(stream, will_write) : nullptr;
}

// An array a kernel writes (or may write).
template <typename T>
inline T* gpu_ptr(array& arr, mlxrocm_stream_t stream) {
  return reinterpret_cast<T*>(
      static_cast<char*>(device_ptr(arr.buffer(), stream, /* will_write */ true)) +
      arr.offset());
}

// An array a kernel only reads.
template <typename T>
inline std::conditional_t<std::is_same_v<T, void>, const void*, const T*> gpu_ptr(
    const array& arr,
    mlxrocm_stream_t stream) {
  using P = std::conditional_t<std::is_same_v<T, void>, const void*, const T*>;
  return reinterpret_cast<P>(
      static_cast<const char*>(device_ptr(
          const_cast<array&>(arr).buffer(), stream, /* will_write */ false)) +
      arr.offset());
}

} // namespace mlx::core::rocm
