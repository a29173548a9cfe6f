// completion.cpp -- see completion.h.
#include "completion.h"

#include <stdexcept>
#include <string>

namespace mlx::core::rocm {

void check(int status) {
  if (status == MLXROCM_OK) {
    return;
  }
  std::string msg = mlxrocm_last_error();
  if (status == MLXROCM_INVALID_ARGUMENT) {
    throw std::invalid_argument(msg);
  }
  throw std::runtime_error(msg);
}

CompletionQueue::CompletionQueue() : shared_(std::make_shared<Shared>()) {
  check(mlxrocm_stream_create(&stream_));
  thread_ = std::thread(&CompletionQueue::thread_main, shared_);
}

CompletionQueue::~CompletionQueue() {
  bool drained;
  {
    std::lock_guard<std::mutex> lock(shared_->mtx);
    shared_->stop = true;
    drained = shared_->queue.empty() && !shared_->running;
  }
  shared_->work.notify_one();
  if (drained) {
    thread_.join(); // returns at once: the thread only has to see `stop`
  } else {
    thread_.detach(); // it finishes the batches it holds, then exits
  }
  // The stream is not destroyed: kernels of a detached thread's batches may
  // still run on it, and at process exit the runtime may already be gone.
}

void CompletionQueue::thread_main(std::shared_ptr<Shared> shared) {
  for (;;) {
    Batch batch;
    {
      std::unique_lock<std::mutex> lock(shared->mtx);
      shared->work.wait(lock, [&] { return !shared->queue.empty() || shared->stop; });
      if (shared->queue.empty()) {
        return; // stop, and nothing left to finish
      }
      batch = std::move(shared->queue.front());
      shared->queue.pop_front();
      shared->running = true;
    }
    // (a batch without an event was committed after the stream had been waited for)
    int rc = batch.event != nullptr ? mlxrocm_event_synchronize(batch.event) : MLXROCM_OK;
    std::string message;
    if (rc != MLXROCM_OK) {
      message = mlxrocm_last_error();
    }
    // Handlers run even after an error: they balance task counters that the
    // evaluating thread may be blocked on.  One that throws must not end the
    // process from this thread: its message reaches the next commit instead.
    for (auto& fn : batch.handlers) {
      try {
        fn();
      } catch (const std::exception& e) {
        if (rc == MLXROCM_OK) {
          rc = MLXROCM_HIP_ERROR;
          message = std::string("a completion handler threw: ") + e.what();
        }
      } catch (...) {
        if (rc == MLXROCM_OK) {
          rc = MLXROCM_HIP_ERROR;
          message = "a completion handler threw";
        }
      }
    }
    batch.handlers.clear();
    batch.retained.clear(); // may free buffers: outside the lock
    if (batch.event != nullptr) {
      (void)mlxrocm_event_destroy(batch.event);
    }
    {
      std::lock_guard<std::mutex> lock(shared->mtx);
      shared->running = false;
      if (rc != MLXROCM_OK && shared->error == MLXROCM_OK) {
        shared->error = rc;
        shared->message = std::move(message);
      }
      if (shared->queue.empty()) {
        shared->idle.notify_all();
      }
    }
  }
}

void CompletionQueue::rethrow_thread_error() {
  int rc;
  std::string message;
  {
    std::lock_guard<std::mutex> lock(shared_->mtx);
    rc = shared_->error;
    message = std::move(shared_->message);
    shared_->error = MLXROCM_OK;
    shared_->message.clear();
  }
  if (rc != MLXROCM_OK) {
    throw std::runtime_error("[rocm] a stream's work failed: " + message);
  }
}

void CompletionQueue::commit() {
  if (!has_pending()) {
    rethrow_thread_error();
    return;
  }
  // The batch is handed to the completion thread whatever fails below: its
  // handlers balance task counters that the evaluating thread may block on
  // (scheduler::wait_for_one), so they must run even when this call throws.
  Batch batch;
  batch.retained = std::move(retained_);
  batch.handlers = std::move(handlers_);
  retained_.clear();
  handlers_.clear();
  std::string failure;
  int rc = mlxrocm_event_create_blocking(&batch.event);
  if (rc == MLXROCM_OK) {
    rc = mlxrocm_event_record(batch.event, stream_);
    if (rc != MLXROCM_OK) {
      failure = mlxrocm_last_error();
      (void)mlxrocm_event_destroy(batch.event);
      batch.event = nullptr;
    }
  } else {
    failure = mlxrocm_last_error();
    batch.event = nullptr;
  }
  if (batch.event == nullptr) {
    // no event to wait for: the buffers may only be dropped once the stream is idle
    (void)mlxrocm_stream_synchronize(stream_);
  }
  {
    std::lock_guard<std::mutex> lock(shared_->mtx);
    shared_->queue.push_back(std::move(batch));
  }
  shared_->work.notify_one();
  if (rc != MLXROCM_OK) {
    if (rc == MLXROCM_INVALID_ARGUMENT) {
      throw std::invalid_argument(failure);
    }
    throw std::runtime_error(failure);
  }
  rethrow_thread_error();
}

void CompletionQueue::synchronize() {
  commit();
  {
    std::unique_lock<std::mutex> lock(shared_->mtx);
    shared_->idle.wait(lock, [&] { return shared_->queue.empty() && !shared_->running; });
  }
  // Work enqueued without anything to retain has no batch: wait for it too.
  check(mlxrocm_stream_synchronize(stream_));
  rethrow_thread_error();
}

} // namespace mlx::core::rocm
