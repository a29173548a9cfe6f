// mock_abi.cpp -- the part of the C ABI (include/mlx_rocm_qmm.h) that the
// backend's host cores call, implemented with host memory and threads so that
// the cores can run, under sanitizers, on a machine without a GPU.
//
// A stream is a thread that runs queued closures in order; the null stream is
// one more such thread.  "Device" memory is malloc'd host memory, copies are
// memcpy closures on the stream, an event completes when the marker closure
// that event_record queued has run.  Nothing here is shipped: only tests link it.
#include "mock_abi.h"

#include <atomic>
#include <condition_variable>
#include <cstdlib>
#include <cstring>
#include <deque>
#include <memory>
#include <mutex>
#include <set>
#include <string>
#include <thread>
#include <vector>

namespace {

struct MockStream {
  std::mutex mtx;
  std::condition_variable cv;
  std::condition_variable drained;
  std::deque<std::function<void()>> queue;
  bool busy{false};
  bool stop{false};
  std::thread thread;

  MockStream() {
    thread = std::thread([this] { run(); });
  }
  ~MockStream() {
    {
      std::lock_guard<std::mutex> lock(mtx);
      stop = true;
    }
    cv.notify_all();
    thread.join();
  }
  void run() {
    for (;;) {
      std::function<void()> fn;
      {
        std::unique_lock<std::mutex> lock(mtx);
        cv.wait(lock, [&] { return !queue.empty() || stop; });
        if (queue.empty()) {
          return;
        }
        fn = std::move(queue.front());
        queue.pop_front();
        busy = true;
      }
      fn();
      {
        std::lock_guard<std::mutex> lock(mtx);
        busy = false;
        if (queue.empty()) {
          drained.notify_all();
        }
      }
    }
  }
  void push(std::function<void()> fn) {
    {
      std::lock_guard<std::mutex> lock(mtx);
      queue.push_back(std::move(fn));
    }
    cv.notify_one();
  }
  void synchronize() {
    std::unique_lock<std::mutex> lock(mtx);
    drained.wait(lock, [&] { return queue.empty() && !busy; });
  }
};

struct MockEvent {
  std::mutex mtx;
  std::condition_variable cv;
  uint64_t recorded{0};
  uint64_t completed{0};
};

struct Registry {
  std::mutex mtx;
  std::set<MockStream*> streams;
  std::unique_ptr<MockStream> null_stream;
  std::atomic<long> device_allocs{0}, host_allocs{0}, events{0};
  std::atomic<long> h2d{0}, d2h{0}, syncs{0};
  std::atomic<int> fail_event_sync{0};
  std::atomic<int> fail_event_record{0};
};

Registry& reg() {
  static Registry* r = new Registry; // outlives static destructors of the tests
  return *r;
}

thread_local std::string g_error;

int fail(int status, const char* msg) {
  g_error = msg;
  return status;
}

MockStream* resolve(mlxrocm_stream_t s) {
  if (s != nullptr) {
    return static_cast<MockStream*>(s);
  }
  auto& r = reg();
  std::lock_guard<std::mutex> lock(r.mtx);
  if (!r.null_stream) {
    r.null_stream = std::make_unique<MockStream>();
  }
  return r.null_stream.get();
}

} // namespace

void mock_launch(mlxrocm_stream_t stream, std::function<void()> fn) {
  resolve(stream)->push(std::move(fn));
}

MockCounters mock_counters() {
  auto& r = reg();
  std::lock_guard<std::mutex> lock(r.mtx);
  return MockCounters{
      r.device_allocs.load(), r.host_allocs.load(), r.events.load(),
      static_cast<long>(r.streams.size()), r.h2d.load(), r.d2h.load(), r.syncs.load()};
}

void mock_fail_event_synchronize(int n) {
  reg().fail_event_sync.store(n);
}

void mock_fail_event_record(int n) {
  reg().fail_event_record.store(n);
}

void mock_shutdown() {
  auto& r = reg();
  std::vector<MockStream*> streams;
  {
    std::lock_guard<std::mutex> lock(r.mtx);
    streams.assign(r.streams.begin(), r.streams.end());
    r.streams.clear();
  }
  for (auto* s : streams) {
    s->synchronize();
    delete s;
  }
  std::unique_ptr<MockStream> null_stream;
  {
    std::lock_guard<std::mutex> lock(r.mtx);
    null_stream = std::move(r.null_stream);
  }
  if (null_stream) {
    null_stream->synchronize();
  }
}

extern "C" {

int mlxrocm_abi_version(void) {
  return MLXROCM_ABI_VERSION;
}
const char* mlxrocm_last_error(void) {
  return g_error.c_str();
}

int mlxrocm_malloc(void** ptr, size_t size) {
  if (ptr == nullptr) {
    return fail(MLXROCM_INVALID_ARGUMENT, "[mock malloc] null result pointer");
  }
  if (size > (size_t(1) << 40)) {
    return fail(MLXROCM_OUT_OF_MEMORY, "[mock malloc] out of memory");
  }
  *ptr = std::malloc(size ? size : 1);
  reg().device_allocs++;
  return MLXROCM_OK;
}
int mlxrocm_free(void* ptr) {
  if (ptr != nullptr) {
    std::free(ptr);
    reg().device_allocs--;
  }
  return MLXROCM_OK;
}
int mlxrocm_host_malloc(void** ptr, size_t size) {
  *ptr = std::malloc(size ? size : 1);
  reg().host_allocs++;
  return MLXROCM_OK;
}
int mlxrocm_host_free(void* ptr) {
  if (ptr != nullptr) {
    std::free(ptr);
    reg().host_allocs--;
  }
  return MLXROCM_OK;
}

static int queue_copy(void* dst, const void* src, size_t n, mlxrocm_stream_t s) {
  resolve(s)->push([=] { std::memcpy(dst, src, n); });
  return MLXROCM_OK;
}
int mlxrocm_memcpy_h2d(void* dst, const void* src, size_t n, mlxrocm_stream_t s) {
  reg().h2d++;
  return queue_copy(dst, src, n, s);
}
int mlxrocm_memcpy_d2h(void* dst, const void* src, size_t n, mlxrocm_stream_t s) {
  reg().d2h++;
  return queue_copy(dst, src, n, s);
}
int mlxrocm_memcpy_d2d(void* dst, const void* src, size_t n, mlxrocm_stream_t s) {
  return queue_copy(dst, src, n, s);
}

int mlxrocm_stream_create(mlxrocm_stream_t* stream) {
  auto* s = new MockStream;
  {
    std::lock_guard<std::mutex> lock(reg().mtx);
    reg().streams.insert(s);
  }
  *stream = s;
  return MLXROCM_OK;
}
int mlxrocm_stream_destroy(mlxrocm_stream_t stream) {
  auto* s = static_cast<MockStream*>(stream);
  if (s == nullptr) {
    return MLXROCM_OK;
  }
  {
    std::lock_guard<std::mutex> lock(reg().mtx);
    reg().streams.erase(s);
  }
  s->synchronize();
  delete s;
  return MLXROCM_OK;
}
int mlxrocm_stream_synchronize(mlxrocm_stream_t stream) {
  reg().syncs++;
  resolve(stream)->synchronize();
  return MLXROCM_OK;
}

int mlxrocm_event_create(mlxrocm_event_t* event) {
  *event = new MockEvent;
  reg().events++;
  return MLXROCM_OK;
}
int mlxrocm_event_create_blocking(mlxrocm_event_t* event) {
  return mlxrocm_event_create(event);
}
int mlxrocm_event_destroy(mlxrocm_event_t event) {
  if (event != nullptr) {
    delete static_cast<MockEvent*>(event);
    reg().events--;
  }
  return MLXROCM_OK;
}
int mlxrocm_event_record(mlxrocm_event_t event, mlxrocm_stream_t stream) {
  int left = reg().fail_event_record.load();
  while (left > 0 && !reg().fail_event_record.compare_exchange_weak(left, left - 1)) {
  }
  if (left > 0) {
    return fail(MLXROCM_HIP_ERROR, "[mock] hipEventRecord failed");
  }
  auto* e = static_cast<MockEvent*>(event);
  uint64_t gen;
  {
    std::lock_guard<std::mutex> lock(e->mtx);
    gen = ++e->recorded;
  }
  resolve(stream)->push([e, gen] {
    std::lock_guard<std::mutex> lock(e->mtx);
    if (gen > e->completed) {
      e->completed = gen;
    }
    e->cv.notify_all();
  });
  return MLXROCM_OK;
}
int mlxrocm_event_wait(mlxrocm_event_t event, mlxrocm_stream_t stream) {
  auto* e = static_cast<MockEvent*>(event);
  uint64_t gen;
  {
    std::lock_guard<std::mutex> lock(e->mtx);
    gen = e->recorded;
  }
  resolve(stream)->push([e, gen] {
    std::unique_lock<std::mutex> lock(e->mtx);
    e->cv.wait(lock, [&] { return e->completed >= gen; });
  });
  return MLXROCM_OK;
}
int mlxrocm_event_synchronize(mlxrocm_event_t event) {
  auto* e = static_cast<MockEvent*>(event);
  {
    std::unique_lock<std::mutex> lock(e->mtx);
    const uint64_t gen = e->recorded;
    e->cv.wait(lock, [&] { return e->completed >= gen; });
  }
  int left = reg().fail_event_sync.load();
  while (left > 0 && !reg().fail_event_sync.compare_exchange_weak(left, left - 1)) {
  }
  if (left > 0) {
    return fail(MLXROCM_HIP_ERROR, "[mock] hipEventSynchronize failed");
  }
  return MLXROCM_OK;
}
int mlxrocm_event_query(mlxrocm_event_t event) {
  auto* e = static_cast<MockEvent*>(event);
  std::lock_guard<std::mutex> lock(e->mtx);
  return e->completed >= e->recorded ? 1 : 0;
}

} // extern "C"
