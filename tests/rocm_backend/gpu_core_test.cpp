// gpu_core_test.cpp -- the ROCm backend's host cores against the real library
// on a GPU: the same completion queue, signal and buffer residency code that
// core_test.cpp runs against the mock, here with HIP streams, blocking events,
// pinned mirrors and the copy kernels of the C ABI as the enqueued work.
// Built by mlx_amd/_build.py (build_glue_gpu_test) and run by
// tests/test_gpu_rocm_backend_cores.py.
#include <unistd.h>

#include <atomic>
#include <condition_variable>
#include <cstdio>
#include <cstdlib>
#include <memory>
#include <mutex>
#include <thread>
#include <vector>

#include "completion.h"
#include "residency.h"
#include "signal.h"

using namespace mlx::core::rocm;

#define CHECK(cond)                                                        \
  do {                                                                     \
    if (!(cond)) {                                                         \
      std::fprintf(stderr, "%s:%d: CHECK failed: %s\n", __FILE__, __LINE__, #cond); \
      std::exit(1);                                                        \
    }                                                                      \
  } while (0)

namespace {

void test_residency_round_trip() {
  CompletionQueue q;
  constexpr int n = 1 << 16;
  auto ints = std::make_shared<RocmBuffer>(n * sizeof(int32_t));
  auto floats = std::make_shared<RocmBuffer>(n * sizeof(float));
  int32_t* h = static_cast<int32_t*>(ints->host_access());
  for (int i = 0; i < n; ++i) {
    h[i] = i - 1000;
  }
  // A second CPU access keeps what the CPU wrote.
  CHECK(static_cast<int32_t*>(ints->host_access())[5] == 5 - 1000);
  // int32 -> float32 on the GPU
  const void* src = ints->device_access(q.stream(), false);
  void* dst = floats->device_access(q.stream(), true);
  check(mlxrocm_copy_contiguous(src, MLXROCM_INT32, dst, MLXROCM_FLOAT32, n, 0, q.stream()));
  q.retain(ints);
  q.retain(floats);
  q.commit();
  // The CPU asks for the result: waits for the kernel, downloads.
  const float* out = static_cast<const float*>(floats->host_access());
  for (int i = 0; i < n; ++i) {
    CHECK(out[i] == static_cast<float>(i - 1000));
  }
  // The CPU changes the source; the next kernel sees the change.
  h = static_cast<int32_t*>(ints->host_access());
  h[0] = 77;
  src = ints->device_access(q.stream(), false);
  dst = floats->device_access(q.stream(), true);
  check(mlxrocm_copy_contiguous(src, MLXROCM_INT32, dst, MLXROCM_FLOAT32, n, 0, q.stream()));
  out = static_cast<const float*>(floats->host_access());
  CHECK(out[0] == 77.0f && out[1] == -999.0f);
  q.synchronize();
}

void test_many_tasks_complete_without_a_later_commit() {
  CompletionQueue q;
  constexpr int n = 1 << 20;
  auto a = std::make_shared<RocmBuffer>(n * sizeof(float));
  auto b = std::make_shared<RocmBuffer>(n * sizeof(float));
  void* pa = a->device_access(q.stream(), true);
  void* pb = b->device_access(q.stream(), true);
  std::mutex mtx;
  std::condition_variable cv;
  int active = 0;
  int completed = 0;
  for (int i = 0; i < 300; ++i) {
    check(mlxrocm_copy_contiguous(pa, MLXROCM_FLOAT32, pb, MLXROCM_BFLOAT16, n, 0, q.stream()));
    {
      std::lock_guard<std::mutex> lock(mtx);
      ++active;
    }
    q.retain(a);
    q.on_complete([&] {
      {
        std::lock_guard<std::mutex> lock(mtx);
        --active;
        ++completed;
      }
      cv.notify_all();
    });
    q.commit();
    std::unique_lock<std::mutex> lock(mtx);
    if (active > 10) { // what eval does above MAX_ACTIVE_TASKS
      const int seen = active;
      cv.wait(lock, [&] { return active < seen; });
    }
  }
  {
    // No synchronize(): the completion thread alone brings this to zero.
    std::unique_lock<std::mutex> lock(mtx);
    cv.wait(lock, [&] { return active == 0; });
  }
  CHECK(completed == 300);
  q.synchronize();
}

void test_signal_orders_two_streams() {
  CompletionQueue producer, consumer;
  constexpr int n = 1 << 22;
  RocmBuffer src(n * sizeof(int32_t)), mid(n * sizeof(int32_t)), dst(n * sizeof(int64_t));
  int32_t* h = static_cast<int32_t*>(src.host_access());
  for (int i = 0; i < n; ++i) {
    h[i] = i;
  }
  Signal sig;
  // The consumer asks first, from another thread, before anything is signalled.
  std::thread requester([&] {
    sig.wait_on_stream(consumer.stream(), 1);
    const void* m = mid.device_access(consumer.stream(), false);
    void* d = dst.device_access(consumer.stream(), true);
    check(mlxrocm_copy_contiguous(m, MLXROCM_INT32, d, MLXROCM_INT64, n, 0, consumer.stream()));
  });
  const void* s = src.device_access(producer.stream(), false);
  void* m = mid.device_access(producer.stream(), true);
  // a few passes so that the producer is still busy when the signal is issued
  for (int pass = 0; pass < 20; ++pass) {
    check(mlxrocm_copy_contiguous(s, MLXROCM_INT32, m, MLXROCM_FLOAT32, n, 0, producer.stream()));
  }
  check(mlxrocm_copy_contiguous(s, MLXROCM_INT32, m, MLXROCM_INT32, n, 0, producer.stream()));
  sig.signal_on_stream(producer.stream(), 1);
  requester.join();
  sig.wait(1);
  CHECK(sig.is_signaled(1));
  const int64_t* out = static_cast<const int64_t*>(dst.host_access());
  for (int i = 0; i < n; i += 4097) {
    CHECK(out[i] == i);
  }
  producer.synchronize();
  consumer.synchronize();
}

} // namespace

int main() {
  alarm(120);
  if (mlxrocm_device_count() < 1) {
    std::fprintf(stderr, "no GPU\n");
    return 2;
  }
  std::puts("residency");
  std::fflush(stdout);
  test_residency_round_trip();
  std::puts("many tasks");
  std::fflush(stdout);
  test_many_tasks_complete_without_a_later_commit();
  std::puts("two streams");
  std::fflush(stdout);
  test_signal_orders_two_streams();
  std::puts("rocm backend cores on the GPU: all tests passed");
  return 0;
}
