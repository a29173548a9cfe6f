// event.cpp -- mlx::core::Event over HIP events of the C ABI
// (interface: mlx/event.h:12-90; CUDA counterpart: mlx/backend/cuda/event.cu:330-409).
//
// A GPU-stream event is a HIP event recorded behind the stream's work; a
// CPU-stream signal/wait runs as a task of that stream's scheduler thread, as
// the other backends do.
#include <atomic>
#include <stdexcept>

#include "mlx/event.h"
#include "mlx/scheduler.h"

#include "device.h"

namespace mlx::core {

namespace rocm {

struct EventImpl {
  mlxrocm_event_t event{nullptr};
  std::atomic<bool> recorded{false};
  std::atomic<Error*> error{nullptr};

  EventImpl() {
    check(mlxrocm_event_create(&event));
  }
  ~EventImpl() {
    (void)mlxrocm_event_destroy(event);
  }
};

} // namespace rocm

Event::Event(Stream s) : stream_(s) {
  event_ = std::make_shared<rocm::EventImpl>();
}

void Event::wait() {
  check_error();
  auto& ev = cast<rocm::EventImpl>();
  if (ev.recorded.load()) {
    rocm::check(mlxrocm_event_synchronize(ev.event));
  }
}

void Event::wait(Stream s) {
  if (s.device == Device::cpu) {
    scheduler::enqueue(s, [*this]() mutable { wait(); });
    return;
  }
  auto& ev = cast<rocm::EventImpl>();
  if (ev.recorded.load()) {
    auto& enc = rocm::get_command_encoder(s);
    rocm::check(mlxrocm_event_wait(ev.event, enc.stream()));
  }
}

void Event::signal(Stream s) {
  auto& ev = cast<rocm::EventImpl>();
  if (s.device == Device::cpu) {
    // Recorded on the null stream from the CPU stream's thread: everything the
    // CPU task produced is already in host memory at that point.
    scheduler::enqueue(s, [*this]() mutable {
      auto& e = cast<rocm::EventImpl>();
      rocm::check(mlxrocm_event_record(e.event, nullptr));
      e.recorded.store(true);
    });
    return;
  }
  auto& enc = rocm::get_command_encoder(s);
  rocm::check(mlxrocm_event_record(ev.event, enc.stream()));
  ev.recorded.store(true);
}

bool Event::is_signaled() const {
  auto& ev = cast<rocm::EventImpl>();
  if (!ev.recorded.load()) {
    return false;
  }
  int done = mlxrocm_event_query(ev.event);
  if (done < 0) {
    rocm::check(done);
  }
  return done == 1;
}

std::atomic<Error*>& Event::error() {
  return cast<rocm::EventImpl>().error;
}

} // namespace mlx::core
