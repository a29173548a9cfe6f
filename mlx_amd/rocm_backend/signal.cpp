// signal.cpp -- see signal.h.
#include "signal.h"

#include "completion.h" // check()

namespace mlx::core::rocm {

Signal::Signal() {
  check(mlxrocm_event_create_blocking(&event_));
}

Signal::~Signal() {
  (void)mlxrocm_event_destroy(event_);
}

void Signal::signal_on_stream(mlxrocm_stream_t stream, uint64_t value) {
  std::lock_guard<std::mutex> lock(mtx_);
  // Recorded under the lock so that a waiter that sees `issued_` also sees
  // this record, not an older one.
  check(mlxrocm_event_record(event_, stream));
  on_gpu_ = true;
  if (value > issued_) {
    issued_ = value;
  }
  issued_cv_.notify_all();
}

void Signal::signal_from_host(uint64_t value) {
  std::lock_guard<std::mutex> lock(mtx_);
  if (value > issued_) {
    issued_ = value;
  }
  issued_cv_.notify_all();
}

void Signal::wait(uint64_t value) {
  bool on_gpu;
  {
    std::unique_lock<std::mutex> lock(mtx_);
    issued_cv_.wait(lock, [&] { return issued_ >= value; });
    on_gpu = on_gpu_;
  }
  if (on_gpu) {
    // A later signal may have re-recorded the event; waiting for that one
    // instead is still correct, records on one stream complete in order.
    check(mlxrocm_event_synchronize(event_));
  }
}

void Signal::wait_on_stream(mlxrocm_stream_t stream, uint64_t value) {
  std::unique_lock<std::mutex> lock(mtx_);
  issued_cv_.wait(lock, [&] { return issued_ >= value; });
  if (on_gpu_) {
    check(mlxrocm_event_wait(event_, stream));
  }
}

bool Signal::is_signaled(uint64_t value) {
  std::lock_guard<std::mutex> lock(mtx_);
  if (issued_ < value) {
    return false;
  }
  if (!on_gpu_) {
    return true;
  }
  int done = mlxrocm_event_query(event_);
  if (done < 0) {
    check(done);
  }
  return done == 1;
}

} // namespace mlx::core::rocm
