// core_test.cpp -- runs the ROCm backend's host cores (completion queue, signal,
// buffer residency) against the host mock of the C ABI.  Built and run by
// tests/test_rocm_backend_cores.py with AddressSanitizer + UBSan and with
// ThreadSanitizer.  Every wait in here is bounded by the alarm in main(): a
// deadlock ends the run with SIGALRM instead of hanging the suite.
#include <unistd.h>

#include <atomic>
#include <chrono>
#include <condition_variable>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <mutex>
#include <stdexcept>
#include <thread>
#include <vector>

#include "completion.h"
#include "mock_abi.h"
#include "residency.h"
#include "signal.h"

using namespace mlx::core::rocm;
using namespace std::chrono_literals;

#define CHECK(cond)                                                        \
  do {                                                                     \
    if (!(cond)) {                                                         \
      std::fprintf(stderr, "%s:%d: CHECK failed: %s\n", __FILE__, __LINE__, #cond); \
      std::exit(1);                                                        \
    }                                                                      \
  } while (0)

namespace {

// What mlx::core::scheduler does for its task counter
// (mlx/scheduler.h:36-63): eval blocks in wait_for_one() when too many tasks
// are active, and only a completion handler can wake it.
struct TaskCounter {
  std::mutex mtx;
  std::condition_variable cv;
  int active{0};
  void notify_new_task() {
    std::lock_guard<std::mutex> lock(mtx);
    ++active;
  }
  void notify_task_completion() {
    {
      std::lock_guard<std::mutex> lock(mtx);
      --active;
    }
    cv.notify_all();
  }
  void wait_for_one() {
    std::unique_lock<std::mutex> lock(mtx);
    const int seen = active;
    cv.wait(lock, [&] { return active < seen; });
  }
  int n_active() {
    std::lock_guard<std::mutex> lock(mtx);
    return active;
  }
};

void test_retained_objects_outlive_the_kernel() {
  CompletionQueue q;
  std::atomic<bool> kernel_done{false};
  std::atomic<bool> released{false};
  std::atomic<bool> released_early{false};
  {
    std::shared_ptr<void> keep(new int(7), [&](void* p) {
      if (!kernel_done.load()) {
        released_early = true;
      }
      released = true;
      delete static_cast<int*>(p);
    });
    mock_launch(q.stream(), [&] {
      std::this_thread::sleep_for(30ms);
      kernel_done = true;
    });
    q.retain(std::move(keep));
  }
  CHECK(q.has_pending());
  q.commit();
  CHECK(!q.has_pending());
  // No further call into the queue: the completion thread alone must notice.
  while (!released.load()) {
    std::this_thread::sleep_for(1ms);
  }
  CHECK(kernel_done.load());
  CHECK(!released_early.load());
  q.synchronize();
}

void test_more_than_ten_active_tasks_do_not_deadlock() {
  constexpr int kMaxActive = 10; // MAX_ACTIVE_TASKS, mlx/transforms.cpp:25
  CompletionQueue q;
  TaskCounter tasks;
  std::atomic<int> completed{0};
  std::vector<int> order;
  std::mutex order_mtx;
  for (int i = 0; i < 200; ++i) {
    mock_launch(q.stream(), [] { std::this_thread::sleep_for(200us); });
    tasks.notify_new_task();
    q.on_complete([&, i] {
      {
        std::lock_guard<std::mutex> lock(order_mtx);
        order.push_back(i);
      }
      ++completed;
      tasks.notify_task_completion();
    });
    q.commit();
    if (tasks.n_active() > kMaxActive) {
      tasks.wait_for_one(); // only the completion thread can release this
    }
  }
  q.synchronize();
  CHECK(completed.load() == 200);
  CHECK(tasks.n_active() == 0);
  for (int i = 0; i < 200; ++i) {
    CHECK(order[i] == i); // handlers run in commit order
  }
}

void test_synchronize_waits_for_unbatched_work_too() {
  CompletionQueue q;
  std::atomic<bool> done{false};
  mock_launch(q.stream(), [&] {
    std::this_thread::sleep_for(20ms);
    done = true;
  });
  q.synchronize(); // nothing retained, no handler: still has to wait
  CHECK(done.load());
}

void test_completion_error_reaches_the_caller_and_handlers_still_run() {
  CompletionQueue q;
  std::atomic<bool> handler_ran{false};
  mock_fail_event_synchronize(1);
  q.on_complete([&] { handler_ran = true; });
  q.commit();
  bool threw = false;
  try {
    q.synchronize();
  } catch (const std::runtime_error& e) {
    threw = std::strstr(e.what(), "hipEventSynchronize") != nullptr;
  }
  CHECK(threw);
  CHECK(handler_ran.load());
  q.synchronize(); // the error was consumed
}

void test_failed_commit_still_runs_the_handlers() {
  // eval() counts the task before it commits (scheduler::notify_new_task), so a
  // commit that cannot record its event must still hand the handlers over, or
  // wait_for_one() would block for good.
  CompletionQueue q;
  TaskCounter tasks;
  std::atomic<bool> kernel_done{false};
  mock_launch(q.stream(), [&] {
    std::this_thread::sleep_for(10ms);
    kernel_done = true;
  });
  tasks.notify_new_task();
  q.on_complete([&] { tasks.notify_task_completion(); });
  mock_fail_event_record(1);
  bool threw = false;
  try {
    q.commit();
  } catch (const std::runtime_error& e) {
    threw = std::strstr(e.what(), "hipEventRecord") != nullptr;
  }
  CHECK(threw);
  // no later commit: the handler has to arrive by itself, behind the kernel
  for (int i = 0; i < 200 && tasks.n_active() != 0; ++i) {
    std::this_thread::sleep_for(5ms);
  }
  CHECK(tasks.n_active() == 0);
  CHECK(kernel_done.load());
  q.synchronize();
}

void test_throwing_handler_is_reported_not_fatal() {
  CompletionQueue q;
  std::atomic<bool> second_ran{false};
  q.on_complete([] { throw std::runtime_error("handler failure"); });
  q.on_complete([&] { second_ran = true; });
  q.commit();
  bool threw = false;
  try {
    q.synchronize();
  } catch (const std::runtime_error& e) {
    threw = std::strstr(e.what(), "handler failure") != nullptr;
  }
  CHECK(threw);
  CHECK(second_ran.load());
  q.synchronize();
}

void test_queue_destroyed_with_work_in_flight() {
  std::atomic<bool> released{false};
  {
    CompletionQueue q;
    mock_launch(q.stream(), [] { std::this_thread::sleep_for(30ms); });
    q.retain(std::shared_ptr<void>(new int(1), [&](void* p) {
      delete static_cast<int*>(p);
      released = true;
    }));
    q.commit();
  } // the detached thread finishes the batch
  while (!released.load()) {
    std::this_thread::sleep_for(1ms);
  }
}

void test_signal_issued_before_and_after_the_wait() {
  mlxrocm_stream_t s = nullptr;
  check(mlxrocm_stream_create(&s));
  // signal first, wait later
  {
    Signal sig;
    std::atomic<bool> done{false};
    mock_launch(s, [&] {
      std::this_thread::sleep_for(20ms);
      done = true;
    });
    CHECK(!sig.is_signaled(1));
    sig.signal_on_stream(s, 1);
    sig.wait(1);
    CHECK(done.load());
    CHECK(sig.is_signaled(1));
    CHECK(!sig.is_signaled(2));
  }
  // wait first: the waiter may not pass before the signal exists AND the work
  // in front of it has finished
  {
    Signal sig;
    std::atomic<bool> done{false};
    std::atomic<bool> passed{false};
    std::thread waiter([&] {
      sig.wait(1);
      CHECK(done.load());
      passed = true;
    });
    std::this_thread::sleep_for(20ms);
    CHECK(!passed.load());
    mock_launch(s, [&] {
      std::this_thread::sleep_for(20ms);
      done = true;
    });
    sig.signal_on_stream(s, 1);
    waiter.join();
    CHECK(passed.load());
  }
  // a producer on the host (a CPU-stream task)
  {
    Signal sig;
    std::atomic<bool> produced{false};
    std::thread waiter([&] {
      sig.wait(1);
      CHECK(produced.load());
    });
    std::this_thread::sleep_for(10ms);
    produced = true;
    sig.signal_from_host(1);
    waiter.join();
    CHECK(sig.is_signaled(1));
  }
  // a counting fence: value 2 is not satisfied by the first update
  {
    Signal sig;
    std::atomic<int> updates{0};
    std::thread waiter([&] {
      sig.wait(2);
      CHECK(updates.load() == 2);
    });
    mock_launch(s, [&] { updates = 1; });
    sig.signal_on_stream(s, 1);
    std::this_thread::sleep_for(10ms);
    mock_launch(s, [&] {
      std::this_thread::sleep_for(10ms);
      updates = 2;
    });
    sig.signal_on_stream(s, 2);
    waiter.join();
  }
  check(mlxrocm_stream_synchronize(s));
  check(mlxrocm_stream_destroy(s));
}

void test_signal_orders_one_stream_behind_another() {
  mlxrocm_stream_t producer = nullptr, consumer = nullptr;
  check(mlxrocm_stream_create(&producer));
  check(mlxrocm_stream_create(&consumer));
  Signal sig;
  std::atomic<int> value{0};
  std::atomic<int> seen{-1};
  // The consumer's wait is requested from another thread before the producer
  // has signalled: it must block that thread, not skip the wait.
  std::thread requester([&] {
    sig.wait_on_stream(consumer, 1);
    mock_launch(consumer, [&] { seen = value.load(); });
  });
  std::this_thread::sleep_for(10ms);
  mock_launch(producer, [&] {
    std::this_thread::sleep_for(30ms);
    value = 42;
  });
  sig.signal_on_stream(producer, 1);
  requester.join();
  check(mlxrocm_stream_synchronize(consumer));
  CHECK(seen.load() == 42);
  check(mlxrocm_stream_destroy(producer));
  check(mlxrocm_stream_destroy(consumer));
}

void test_residency_transitions() {
  mlxrocm_stream_t s = nullptr;
  check(mlxrocm_stream_create(&s));
  const MockCounters before = mock_counters();
  {
    RocmBuffer buf(3 * sizeof(int));
    // The CPU fills a fresh buffer: nothing to download.
    int* host = static_cast<int*>(buf.host_access());
    host[0] = 1;
    host[1] = 2;
    host[2] = 3;
    CHECK(mock_counters().d2h_copies == before.d2h_copies);
    // A second CPU access must not bring stale device bytes over the writes.
    int* again = static_cast<int*>(buf.host_access());
    CHECK(again == host);
    CHECK(host[0] == 1 && host[1] == 2 && host[2] == 3);
    CHECK(mock_counters().d2h_copies == before.d2h_copies);

    // A kernel reads it: one upload, and only one for two uses.
    int sum = 0;
    const int* dev = static_cast<const int*>(buf.device_access(s, /* will_write */ false));
    mock_launch(s, [&sum, dev] { sum = dev[0] + dev[1] + dev[2]; });
    const int* dev2 = static_cast<const int*>(buf.device_access(s, false));
    CHECK(dev2 == dev);
    check(mlxrocm_stream_synchronize(s));
    CHECK(sum == 6);
    CHECK(mock_counters().h2d_copies == before.h2d_copies + 1);

    // Reading on the GPU left the mirror current: no download.
    host = static_cast<int*>(buf.host_access());
    CHECK(host[2] == 3);
    CHECK(mock_counters().d2h_copies == before.d2h_copies);

    // A kernel writes it: the next CPU access waits for the kernel and downloads.
    int* wdev = static_cast<int*>(buf.device_access(s, /* will_write */ true));
    mock_launch(s, [wdev] {
      std::this_thread::sleep_for(20ms);
      wdev[1] = 20;
    });
    host = static_cast<int*>(buf.host_access());
    CHECK(host[0] == 1 && host[1] == 20 && host[2] == 3);
    CHECK(mock_counters().d2h_copies == before.d2h_copies + 1);

    // CPU writes, GPU reads again: uploaded again, and the CPU's bytes win.
    host[0] = 100;
    dev = static_cast<const int*>(buf.device_access(s, false));
    mock_launch(s, [&sum, dev] { sum = dev[0] + dev[1] + dev[2]; });
    check(mlxrocm_stream_synchronize(s));
    CHECK(sum == 123);
  }
  const MockCounters after = mock_counters();
  CHECK(after.live_device_allocs == before.live_device_allocs);
  CHECK(after.live_host_allocs == before.live_host_allocs);
  check(mlxrocm_stream_destroy(s));
}

void test_host_access_waits_for_readers_on_other_streams() {
  mlxrocm_stream_t writer = nullptr, reader = nullptr;
  check(mlxrocm_stream_create(&writer));
  check(mlxrocm_stream_create(&reader));
  {
    RocmBuffer buf(sizeof(int));
    *static_cast<int*>(buf.host_access()) = 7;
    int* w = static_cast<int*>(buf.device_access(writer, /* will_write */ true));
    mock_launch(writer, [w] { *w = 8; });
    check(mlxrocm_stream_synchronize(writer));
    // a slow kernel on another stream only reads the buffer ...
    std::atomic<bool> read_done{false};
    int seen = 0;
    const int* r = static_cast<const int*>(buf.device_access(reader, false));
    mock_launch(reader, [&, r] {
      std::this_thread::sleep_for(30ms);
      seen = *r;
      read_done = true;
    });
    // ... and the CPU asks for the bytes: it must not get them (and the right to
    // overwrite the device side at the next upload) before that kernel is done
    int* host = static_cast<int*>(buf.host_access());
    CHECK(read_done.load());
    CHECK(seen == 8 && *host == 8);
  }
  check(mlxrocm_stream_destroy(writer));
  check(mlxrocm_stream_destroy(reader));
}

void test_residency_is_safe_from_two_threads() {
  mlxrocm_stream_t s = nullptr;
  check(mlxrocm_stream_create(&s));
  RocmBuffer buf(sizeof(long));
  *static_cast<long*>(buf.host_access()) = 0;
  // A CPU-stream thread and the evaluating thread ask for the buffer at the same
  // time; they only read, the state machine itself must not race.
  std::thread cpu([&] {
    for (int i = 0; i < 200; ++i) {
      CHECK(*static_cast<long*>(buf.host_access()) == 0);
    }
  });
  for (int i = 0; i < 200; ++i) {
    const long* dev = static_cast<const long*>(buf.device_access(s, false));
    mock_launch(s, [dev] { CHECK(*dev == 0); });
  }
  cpu.join();
  check(mlxrocm_stream_synchronize(s));
  check(mlxrocm_stream_destroy(s));
}

} // namespace

int main() {
  alarm(120);
  const MockCounters start = mock_counters();
  test_retained_objects_outlive_the_kernel();
  test_more_than_ten_active_tasks_do_not_deadlock();
  test_synchronize_waits_for_unbatched_work_too();
  test_completion_error_reaches_the_caller_and_handlers_still_run();
  test_failed_commit_still_runs_the_handlers();
  test_throwing_handler_is_reported_not_fatal();
  test_queue_destroyed_with_work_in_flight();
  test_signal_issued_before_and_after_the_wait();
  test_signal_orders_one_stream_behind_another();
  test_residency_transitions();
  test_host_access_waits_for_readers_on_other_streams();
  test_residency_is_safe_from_two_threads();
  std::this_thread::sleep_for(50ms); // let a detached completion thread exit
  mock_shutdown();
  const MockCounters end = mock_counters();
  CHECK(end.live_events == start.live_events);
  CHECK(end.live_device_allocs == start.live_device_allocs);
  CHECK(end.live_host_allocs == start.live_host_allocs);
  std::puts("rocm backend cores: all tests passed");
  return 0;
}
