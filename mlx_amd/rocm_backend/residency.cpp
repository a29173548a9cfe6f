// residency.cpp -- see residency.h.
#include "residency.h"

#include "completion.h" // check()

namespace mlx::core::rocm {

RocmBuffer::RocmBuffer(size_t size) : size_(size) {
  check(mlxrocm_malloc(&device_, size));
}

RocmBuffer::~RocmBuffer() {
  (void)mlxrocm_free(device_);
  (void)mlxrocm_host_free(host_);
}

void* RocmBuffer::device_access(mlxrocm_stream_t stream, bool will_write) {
  std::lock_guard<std::mutex> lock(mtx_);
  // A stale device side means host_access() ran last, and that waited for every
  // stream with work on the buffer: the upload cannot overtake an older kernel.
  if (!device_current_) {
    check(mlxrocm_memcpy_h2d(device_, host_, size_, stream));
    device_current_ = true;
  }
  if (will_write) {
    host_current_ = false;
    last_stream_ = stream;
  } else if (last_stream_ == nullptr) {
    last_stream_ = stream;
  }
  note_pending(stream);
  touched_by_gpu_ = true;
  return device_;
}

void RocmBuffer::note_pending(mlxrocm_stream_t stream) {
  for (mlxrocm_stream_t s : pending_streams_) {
    if (s == stream) {
      return;
    }
  }
  pending_streams_.push_back(stream);
}

void* RocmBuffer::host_access() {
  std::lock_guard<std::mutex> lock(mtx_);
  if (host_ == nullptr) {
    check(mlxrocm_host_malloc(&host_, size_));
  }
  if (!host_current_ && touched_by_gpu_) {
    // Ordered behind the kernels that produced the bytes: the last writer's stream.
    check(mlxrocm_memcpy_d2h(host_, device_, size_, last_stream_));
    note_pending(last_stream_);
  }
  // Every stream that used the buffer since the last host access: writers,
  // readers (the next upload must not overwrite what they still read) and an
  // upload still reading the mirror the caller may now write.
  for (mlxrocm_stream_t s : pending_streams_) {
    check(mlxrocm_stream_synchronize(s));
  }
  pending_streams_.clear();
  host_current_ = true;
  device_current_ = false;
  return host_;
}

} // namespace mlx::core::rocm
