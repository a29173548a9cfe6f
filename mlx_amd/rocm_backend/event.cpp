// event.cpp -- mlx::core::Event for the ROCm backend
// (interface: mlx/event.h:12-90; CUDA counterpart: mlx/backend/cuda/event.cu:330-409).
//
// The state is a rocm::Signal (signal.h): a host counter that says a signal has
// been issued, plus a HIP event when it was issued on a GPU stream.  A waiter
// that comes first blocks until the signal exists; a CPU-stream producer or
// consumer runs as a task of that stream's scheduler thread, as in the other
// backends.
#include <atomic>

#include "mlx/event.h"
#include "mlx/scheduler.h"

#include "device.h"
#include "signal.h"

namespace mlx::core {

namespace rocm {

struct EventImpl {
  Signal signal;
  std::atomic<Error*> error{nullptr};
};

} // namespace rocm

Event::Event(Stream s) : stream_(s) {
  event_ = std::make_shared<rocm::EventImpl>();
}

void Event::wait() {
  check_error();
  cast<rocm::EventImpl>().signal.wait(value());
}

void Event::wait(Stream s) {
  if (s.device == Device::cpu) {
    // The CPU stream's thread blocks, not the caller.
    scheduler::enqueue(s, [*this]() mutable { wait(); });
    return;
  }
  cast<rocm::EventImpl>().signal.wait_on_stream(
      rocm::get_command_encoder(s).stream(), value());
}

void Event::signal(Stream s) {
  if (s.device == Device::cpu) {
    // Runs after the CPU tasks queued so far: what they produced is in host
    // memory by then.
    scheduler::enqueue(s, [*this]() mutable {
      cast<rocm::EventImpl>().signal.signal_from_host(value());
    });
    return;
  }
  cast<rocm::EventImpl>().signal.signal_on_stream(
      rocm::get_command_encoder(s).stream(), value());
}

bool Event::is_signaled() const {
  return cast<rocm::EventImpl>().signal.is_signaled(value());
}

std::atomic<Error*>& Event::error() {
  return cast<rocm::EventImpl>().error;
}

} // namespace mlx::core
