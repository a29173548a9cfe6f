// fence.cpp -- mlx::core::Fence for the ROCm backend (interface:
// mlx/fence.h:9-45; CUDA counterpart: mlx/backend/cuda/fence.cpp:10-42).
//
// A fence counts its updates and a waiter waits for the count it saw: exactly
// the value semantics of mlx::core::Event here (event.cpp), so the fence is an
// event whose value is raised by one per update.  Where the CUDA backend moves
// an array that crosses to the CPU into managed memory at update time, nothing
// is moved here: the CPU side reaches the bytes through Buffer::raw_ptr(), which
// downloads them after the producing stream has finished (residency.h).
#include <cstdint>
#include <mutex>

#include "mlx/event.h"
#include "mlx/fence.h"

namespace mlx::core {

namespace rocm {

struct FenceImpl {
  std::mutex mtx; // update() comes from one thread, wait() from any
  uint64_t count{0};
  Event event;
  explicit FenceImpl(Stream s) : event(s) {}
};

} // namespace rocm

Fence::Fence(Stream s) {
  fence_ = std::make_shared<rocm::FenceImpl>(s);
}

void Fence::update(Stream s, const array&, bool /* cross_device */) {
  auto& f = cast<rocm::FenceImpl>();
  Event e;
  {
    std::lock_guard<std::mutex> lock(f.mtx);
    f.event.set_value(++f.count);
    e = f.event; // shares the state, carries this update's value
  }
  e.signal(s);
}

void Fence::wait(Stream s, const array&) {
  auto& f = cast<rocm::FenceImpl>();
  Event e;
  {
    std::lock_guard<std::mutex> lock(f.mtx);
    e = f.event;
  }
  if (e.value() == 0) {
    return; // never updated
  }
  e.wait(s);
}

} // namespace mlx::core
