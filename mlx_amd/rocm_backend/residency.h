// residency.h -- what an allocator::Buffer of the ROCm backend points at, and
// the rules for which side of the PCIe link holds its current bytes.
//
// MLX's other GPU backends hand out memory that the CPU can simply read: unified
// memory on Metal, managed memory on CUDA (a buffer moves to managed memory the
// first time the CPU asks for it, mlx/backend/cuda/allocator.cpp:392-399).  An
// MI355X buffer lives in HBM and the CPU gets a pinned host mirror on demand.
// Each side has a "holds the current bytes" flag:
//
//   device_access(stream, will_write)   host_access()
//   ---------------------------------   --------------------------------------
//   device stale -> upload on `stream`  host stale -> wait for the GPU work on
//   will_write   -> host becomes stale                the buffer, download
//   remembers `stream`                  device becomes stale (the caller may
//                                       write through the pointer)
//
// A second host_access() with nothing in between finds the mirror current and
// copies nothing, so bytes the CPU wrote are never overwritten by older device
// contents; a kernel that only reads leaves a current mirror current.  Because
// allocator::Buffer::raw_ptr() is the only way MLX's CPU code reaches the data
// and does not say whether it will write, every host access costs one upload at
// the next kernel that touches the buffer -- the analogue of managed pages
// migrating back.  A buffer no kernel has touched yet has nothing to download:
// the CPU filling a new array costs one upload and no download.  The mirror, once made, stays allocated until the buffer is
// freed: pointers that CPU tasks still hold stay valid.
//
// No MLX types appear here: the file builds against a host mock of the C ABI
// for the CPU tests.
#pragma once

#include <cstddef>
#include <mutex>
#include <vector>

#include "mlx_rocm_qmm.h"

namespace mlx::core::rocm {

class RocmBuffer {
 public:
  // Allocates `size` bytes of device memory; throws on failure.
  explicit RocmBuffer(size_t size);
  ~RocmBuffer();
  RocmBuffer(const RocmBuffer&) = delete;
  RocmBuffer& operator=(const RocmBuffer&) = delete;

  size_t size() const {
    return size_;
  }

  // Pointer for kernels enqueued on `stream`.  `will_write` is false for
  // operands a kernel only reads.
  void* device_access(mlxrocm_stream_t stream, bool will_write);
  // Pointer for the CPU; valid until the buffer is freed.
  void* host_access();

 private:
  void note_pending(mlxrocm_stream_t stream);
  std::mutex mtx_;
  size_t size_;
  void* device_{nullptr};
  void* host_{nullptr};
  bool device_current_{true}; // fresh memory: nothing to lose on either side
  bool host_current_{false};
  bool touched_by_gpu_{false}; // false: fresh memory, no bytes worth downloading
  // Streams with work on the buffer that host_access() has not waited for yet
  // (a kernel that only reads may run on another stream than the last writer).
  std::vector<mlxrocm_stream_t> pending_streams_;
  mlxrocm_stream_t last_stream_{nullptr}; // orders the download behind the last writer
};

} // namespace mlx::core::rocm
