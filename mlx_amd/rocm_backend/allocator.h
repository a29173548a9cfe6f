// allocator.h -- buffer record of the ROCm backend and the device-pointer
// accessor eval_gpu bodies use (the counterpart of gpu_ptr<T>,
// mlx/backend/cuda/utils.h:26-39, and cu::CudaBuffer,
// mlx/backend/cuda/allocator.h:18-24).
#pragma once

#include <cstddef>
#include <type_traits>

#include "mlx/array.h"

#include "mlx_rocm_qmm.h"

namespace mlx::core::rocm {

// What allocator::Buffer::ptr() points at.  `device` is HBM; `host` is a pinned
// mirror that exists only after the CPU asked for the data (Buffer::raw_ptr()).
struct RocmBuffer {
  void* device{nullptr};
  void* host{nullptr};
  size_t size{0};
  bool host_dirty{false}; // the CPU may have written `host` since the last upload
};

// Device address of a buffer; uploads a dirty host mirror on `stream` first.
void* device_ptr(allocator::Buffer buffer, mlxrocm_stream_t stream);

template <typename T>
inline T* gpu_ptr(array& arr, mlxrocm_stream_t stream) {
  return reinterpret_cast<T*>(
      static_cast<char*>(device_ptr(arr.buffer(), stream)) + arr.offset());
}

template <typename T>
inline std::conditional_t<std::is_same_v<T, void>, void*, const T*> gpu_ptr(
    const array& arr,
    mlxrocm_stream_t stream) {
  return gpu_ptr<T>(const_cast<array&>(arr), stream);
}

} // namespace mlx::core::rocm
