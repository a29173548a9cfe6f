// device.cpp -- see device.h.
#include "device.h"

#include <mutex>
#include <stdexcept>
#include <string>
#include <unordered_map>

namespace mlx::core::rocm {

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
  auto& local = thread_encoders();
  for (auto& [index, encoder] : local) {
    encoder->synchronize(); // so that each completion thread can be joined
  }
  local.clear();
}

} // namespace mlx::core::rocm
