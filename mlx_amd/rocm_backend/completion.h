// completion.h -- one HIP stream plus the host thread that notices when work
// enqueued on it has finished.
//
// MLX keeps arrays alive and counts active tasks until the GPU is done with
// them, and evaluating blocks in scheduler::wait_for_one() once more than ten
// tasks are in flight (mlx/transforms.cpp:25,271-283): completion therefore has
// to be noticed without any further call from the evaluating thread.  The CUDA
// backend does it with a worker thread woken by a host callback
// (mlx/backend/cuda/worker.cpp:8-88).  Here each commit() records a
// blocking-sync HIP event behind the enqueued kernels and hands {event,
// retained objects, handlers} to this queue's thread, which sleeps in
// hipEventSynchronize, runs the handlers, drops the retained objects and takes
// the next batch -- batches complete in stream order, so one thread per stream
// is enough and the handlers of a stream run in commit order.
//
// No MLX types appear here on purpose: the file builds and runs against a host
// mock of the C ABI for the CPU tests.
#pragma once

#include <condition_variable>
#include <deque>
#include <functional>
#include <memory>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

#include "mlx_rocm_qmm.h"

namespace mlx::core::rocm {

// Throws std::invalid_argument / std::runtime_error for a non-zero status of
// the C ABI (the message is mlxrocm_last_error()).
void check(int status);

class CompletionQueue {
 public:
  CompletionQueue();
  // Work still in flight is left to the (then detached) thread; nothing is
  // waited for, so that tear-down at process exit cannot block.
  ~CompletionQueue();
  CompletionQueue(const CompletionQueue&) = delete;
  CompletionQueue& operator=(const CompletionQueue&) = delete;

  mlxrocm_stream_t stream() const {
    return stream_;
  }

  // Keep `keep` alive until the work enqueued before the next commit() is done.
  void retain(std::shared_ptr<void> keep) {
    retained_.push_back(std::move(keep));
  }
  // Run `fn` on the completion thread once that work is done.
  void on_complete(std::function<void()> fn) {
    handlers_.push_back(std::move(fn));
  }
  bool has_pending() const {
    return !retained_.empty() || !handlers_.empty();
  }

  // Files what retain()/on_complete() collected under an event recorded now.
  // Rethrows an error the completion thread met since the last call.
  void commit();
  // commit(), then block until every committed batch has completed and its
  // handlers have run.
  void synchronize();

 private:
  struct Batch {
    mlxrocm_event_t event{nullptr};
    std::vector<std::shared_ptr<void>> retained;
    std::vector<std::function<void()>> handlers;
  };
  struct Shared {
    std::mutex mtx;
    std::condition_variable work; // a batch arrived, or stop
    std::condition_variable idle; // the queue drained
    std::deque<Batch> queue;
    bool running{false}; // the thread is finishing a batch it has popped
    bool stop{false};
    int error{MLXROCM_OK};
    std::string message;
  };
  static void thread_main(std::shared_ptr<Shared> shared);
  void rethrow_thread_error();

  mlxrocm_stream_t stream_{nullptr};
  std::vector<std::shared_ptr<void>> retained_;
  std::vector<std::function<void()>> handlers_;
  std::shared_ptr<Shared> shared_;
  std::thread thread_;
};

} // namespace mlx::core::rocm
