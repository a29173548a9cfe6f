// device.h -- per-stream command encoder of the ROCm backend.
//
// Part of the `mlx/backend/rocm` tree: host C++ written against MLX's own
// headers, calling HIP only through the C ABI of mlx_rocm_qmm.h.  Plays the
// role of cu::CommandEncoder (mlx/backend/cuda/device.h:21-164) with plain
// stream launches instead of graph batching: eval_gpu bodies enqueue kernels on
// the encoder's stream, and the buffers they touch are kept until the
// encoder's completion thread has seen an event recorded behind those kernels
// (completion.h).
#pragma once

#include <functional>
#include <memory>

#include "mlx/array.h"
#include "mlx/stream.h"

#include "completion.h"

namespace mlx::core::rocm {

class CommandEncoder {
 public:
  explicit CommandEncoder(Stream s) : mlx_stream_(s) {}

  mlxrocm_stream_t stream() const {
    return queue_.stream();
  }

  // Keep `arr`'s buffer (not the array object and its graph) alive until the
  // work enqueued so far has completed.
  void add_temporary(const array& arr) {
    queue_.retain(arr.data_shared_ptr());
  }
  void retain(std::shared_ptr<void> data) {
    queue_.retain(std::move(data));
  }
  void add_completed_handler(std::function<void()> fn) {
    queue_.on_complete(std::move(fn));
  }
  bool needs_commit() const {
    return queue_.has_pending();
  }
  void commit() {
    queue_.commit();
  }
  void synchronize() {
    queue_.synchronize();
  }

 private:
  Stream mlx_stream_;
  CompletionQueue queue_;
};

// Encoder of a GPU stream created by gpu::new_stream on this thread (or by
// gpu::new_thread_unsafe_stream on any thread); throws if there is none
// (mlx/backend/cuda/device.cpp:565-588).
CommandEncoder& get_command_encoder(Stream s);
void new_encoder(Stream s, bool thread_unsafe);
// Drains and drops this thread's encoders.
void clear_encoders();

} // namespace mlx::core::rocm
