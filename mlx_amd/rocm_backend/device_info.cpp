// device_info.cpp -- gpu::is_available / device_count / device_info for the ROCm
// backend (interface: mlx/backend/gpu/device_info.h:13-34).
#include <mutex>
#include <string>
#include <unordered_map>
#include <variant>
#include <vector>

#include "mlx/backend/gpu/device_info.h"

#include "device.h"

namespace mlx::core::gpu {

bool is_available() {
  return mlxrocm_device_count() > 0;
}

int device_count() {
  int n = mlxrocm_device_count();
  return n < 0 ? 0 : n;
}

const std::unordered_map<std::string, std::variant<std::string, size_t>>&
device_info(int device_index) {
  using Info = std::unordered_map<std::string, std::variant<std::string, size_t>>;
  static std::mutex mtx;
  static std::unordered_map<int, Info> cache;
  std::lock_guard<std::mutex> lock(mtx);
  auto it = cache.find(device_index);
  if (it != cache.end()) {
    return it->second;
  }
  char name[256] = {0};
  int compute_units = 0;
  size_t total_memory = 0;
  int clock_khz = 0;
  rocm::check(mlxrocm_device_info(
      device_index, name, &compute_units, &total_memory, &clock_khz));
  Info info;
  info["device_name"] = std::string(name);
  info["architecture"] = std::string("gfx950");
  info["total_memory"] = total_memory;
  info["memory_size"] = total_memory;
  info["compute_units"] = static_cast<size_t>(compute_units);
  info["clock_khz"] = static_cast<size_t>(clock_khz);
  return cache.emplace(device_index, std::move(info)).first->second;
}

} // namespace mlx::core::gpu
