// signal.h -- the state behind mlx::core::Event and mlx::core::Fence: a
// counter that producers raise, on a GPU stream or from the host, and that
// consumers wait for, on the host or on another GPU stream.
//
// An MLX event is signalled "at a value" and may be signalled again at a higher
// one (a Fence counts its updates, mlx/backend/cuda/fence.cpp:35-42); a waiter
// may arrive before the signal has even been issued, e.g. when the producer is
// a task still queued on a CPU stream (mlx/event.h:17-27).  So there are two
// stages: the host-side `issued` counter says a signal for that value has been
// put in place, and, if it was put on a GPU stream, a HIP event recorded at
// that point says when the GPU actually gets there.  Waiters block on the first
// stage with a condition variable and on the second with the HIP event; no
// kernel ever spins on a flag.
//
// No MLX types appear here: the file builds against a host mock of the C ABI
// for the CPU tests.
#pragma once

#include <condition_variable>
#include <cstdint>
#include <mutex>

#include "mlx_rocm_qmm.h"

namespace mlx::core::rocm {

class Signal {
 public:
  Signal();
  ~Signal();
  Signal(const Signal&) = delete;
  Signal& operator=(const Signal&) = delete;

  // The event counts as signalled at `value` once the work enqueued on
  // `stream` so far has completed.
  void signal_on_stream(mlxrocm_stream_t stream, uint64_t value);
  // Signalled at `value` now (the producer ran on the host).
  void signal_from_host(uint64_t value);

  // Block the calling thread until signalled at `value` or higher.
  void wait(uint64_t value);
  // Make work enqueued on `stream` from now on start after the signal at
  // `value`.  Blocks the calling thread only until that signal has been issued.
  void wait_on_stream(mlxrocm_stream_t stream, uint64_t value);
  // True once wait(value) would return without blocking.
  bool is_signaled(uint64_t value);

 private:
  std::mutex mtx_;
  std::condition_variable issued_cv_;
  uint64_t issued_{0};   // highest value a signal has been put in place for
  bool on_gpu_{false};   // event_ carries a record that belongs to issued_
  mlxrocm_event_t event_{nullptr};
};

} // namespace mlx::core::rocm
