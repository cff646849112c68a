// device_handle_t (reference: lib/kernels/include/kernels/device_handle_t.dtg.toml,
// device_handle_t.h): a PerDeviceFFHandle for the GPU, nothing for the CPU.
#pragma once
#include "kernels/ff_handle.h"
#include <variant>

namespace FlexFlow {

struct device_handle_t {
  std::variant<PerDeviceFFHandle, std::monostate> raw;
  static device_handle_t for_gpu(PerDeviceFFHandle const &h) { return device_handle_t{h}; }
  static device_handle_t for_cpu() { return device_handle_t{std::monostate{}}; }
  bool is_for_gpu() const { return raw.index() == 0; }
  bool is_for_cpu() const { return raw.index() == 1; }
  PerDeviceFFHandle const &require_for_gpu() const {
    if (!is_for_gpu()) throw std::runtime_error("device_handle_t: expected for_gpu");
    return std::get<0>(raw);
  }
};

}  // namespace FlexFlow
