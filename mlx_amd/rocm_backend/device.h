// device.h -- per-stream command encoder of the ROCm backend.
//
// Part of the `mlx/backend/rocm` tree: host C++ written against MLX's own
// headers, calling HIP only through the C ABI of mlx_rocm_qmm.h.  Mirrors the
// role of cu::CommandEncoder (mlx/backend/cuda/device.h:21-164) with plain
// stream launches instead of graph batching: eval_gpu bodies enqueue kernels on
// the encoder's stream, arrays they read are retained until an event recorded
// after the launch has completed.
#pragma once

#include <deque>
#include <functional>
#include <mutex>
#include <vector>

#include "mlx/array.h"
#include "mlx/stream.h"

#include "mlx_rocm_qmm.h"

namespace mlx::core::rocm {

// Throws std::runtime_error / std::invalid_argument for a non-zero status of
// the C ABI (the message is mlxrocm_last_error()).
void check(int status);

class CommandEncoder {
 public:
  explicit CommandEncoder(Stream s);
  ~CommandEncoder();
  CommandEncoder(const CommandEncoder&) = delete;
  CommandEncoder& operator=(const CommandEncoder&) = delete;

  mlxrocm_stream_t stream() const {
    return stream_;
  }

  // Keep `arr`'s buffer alive until the work enqueued so far has completed.
  void add_temporary(const array& arr) {
    pending_.push_back(arr);
  }
  void add_completed_handler(std::function<void()> fn) {
    handlers_.push_back(std::move(fn));
  }
  bool needs_commit() const {
    return !pending_.empty() || !handlers_.empty();
  }
  // Records an event behind the enqueued work and files the retained arrays
  // and handlers under it; completed batches are released on later commits and
  // in synchronize().
  void commit();
  void synchronize();

 private:
  struct Batch {
    mlxrocm_event_t event;
    std::vector<array> arrays;
    std::vector<std::function<void()>> handlers;
  };
  void reap(bool wait);

  Stream mlx_stream_;
  mlxrocm_stream_t stream_{nullptr};
  std::vector<array> pending_;
  std::vector<std::function<void()>> handlers_;
  std::deque<Batch> in_flight_;
};

// Encoder of a GPU stream created by gpu::new_stream on this thread (or by
// gpu::new_thread_unsafe_stream on any thread); throws if there is none
// (mlx/backend/cuda/device.cpp:565-588).
CommandEncoder& get_command_encoder(Stream s);
void new_encoder(Stream s, bool thread_unsafe);
void clear_encoders();

} // namespace mlx::core::rocm
