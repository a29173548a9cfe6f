// device.cpp -- see device.h.
#include "device.h"

#include <stdexcept>
#include <string>
#include <unordered_map>

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

CommandEncoder::CommandEncoder(Stream s) : mlx_stream_(s) {
  check(mlxrocm_stream_create(&stream_));
}

CommandEncoder::~CommandEncoder() {
  // Devices are torn down at process exit in an unspecified order: drop the
  // bookkeeping, do not call into the runtime.
}

void CommandEncoder::commit() {
  reap(/* wait */ false);
  if (!needs_commit()) {
    return;
  }
  Batch b;
  check(mlxrocm_event_create(&b.event));
  check(mlxrocm_event_record(b.event, stream_));
  b.arrays = std::move(pending_);
  b.handlers = std::move(handlers_);
  pending_.clear();
  handlers_.clear();
  in_flight_.push_back(std::move(b));
}

void CommandEncoder::reap(bool wait) {
  while (!in_flight_.empty()) {
    Batch& b = in_flight_.front();
    if (wait) {
      check(mlxrocm_event_synchronize(b.event));
    } else {
      int done = mlxrocm_event_query(b.event);
      if (done < 0) {
        check(done);
      }
      if (done == 0) {
        return; // batches complete in order
      }
    }
    for (auto& fn : b.handlers) {
      fn();
    }
    check(mlxrocm_event_destroy(b.event));
    in_flight_.pop_front(); // releases the retained arrays
  }
}

void CommandEncoder::synchronize() {
  commit();
  check(mlxrocm_stream_synchronize(stream_));
  reap(/* wait */ true);
}

namespace {

using EncoderMap = std::unordered_map<int, std::unique_ptr<CommandEncoder>>;

EncoderMap& thread_encoders() {
  static thread_local EncoderMap encoders;
  return encoders;
}

EncoderMap& global_encoders() {
  static EncoderMap* encoders = new EncoderMap; // leaked on purpose
  return *encoders;
}

std::mutex& global_mutex() {
  static std::mutex m;
  return m;
}

} // namespace

void new_encoder(Stream s, bool thread_unsafe) {
  if (thread_unsafe) {
    std::lock_guard<std::mutex> lock(global_mutex());
    global_encoders().try_emplace(s.index, std::make_unique<CommandEncoder>(s));
  } else {
    thread_encoders().try_emplace(s.index, std::make_unique<CommandEncoder>(s));
  }
}

CommandEncoder& get_command_encoder(Stream s) {
  auto& local = thread_encoders();
  if (auto it = local.find(s.index); it != local.end()) {
    return *it->second;
  }
  {
    std::lock_guard<std::mutex> lock(global_mutex());
    auto& global = global_encoders();
    if (auto it = global.find(s.index); it != global.end()) {
      return *it->second;
    }
  }
  throw std::runtime_error(
      "There is no Stream(gpu, " + std::to_string(s.index) + ") in current thread.");
}

void clear_encoders() {
  thread_encoders().clear();
}

} // namespace mlx::core::rocm
