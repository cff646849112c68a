// device_stream_t (reference: lib/kernels/include/kernels/device_stream_t.dtg.toml,
// device_stream_t.h).  Also pulls in device_handle_t and the managed stream /
// handle types, which most callers use together.
#pragma once
#include "kernels/device.h"
#include "kernels/device_handle_t.h"
#include "pcg/device_type.h"
#include <cstddef>
#include <variant>

namespace FlexFlow {

struct device_stream_t {
  std::variant<ffStream_t, std::monostate> raw;
  static device_stream_t gpu(ffStream_t s) { return device_stream_t{s}; }
  static device_stream_t cpu() { return device_stream_t{std::monostate{}}; }
  bool is_gpu() const { return raw.index() == 0; }
  bool is_cpu() const { return raw.index() == 1; }
  ffStream_t require_gpu() const {
    if (!is_gpu()) throw std::runtime_error("device_stream_t: expected gpu");
    return std::get<0>(raw);
  }
};

device_stream_t get_gpu_device_stream();
device_stream_t get_cpu_device_stream();
device_stream_t get_stream_for_device_type(DeviceType);

}  // namespace FlexFlow
#include "kernels/managed_ff_stream.h"
#include "kernels/managed_per_device_ff_handle.h"
