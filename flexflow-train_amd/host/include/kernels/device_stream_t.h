// device_stream_t / device_handle_t variants (reference:
// lib/kernels/include/kernels/device_stream_t.dtg.toml, device_handle_t.dtg.toml,
// device_stream_t.h, ff_handle.h:12-24).
#pragma once
#include "kernels/device.h"
#include "pcg/device_type.h"
#include <cstddef>
#include <variant>

namespace FlexFlow {

struct PerDeviceFFHandle {
  ffHandle_t dnn;        // null: no vendor library behind these kernels
  ffblasHandle_t blas;   // null
  void *workSpace;
  size_t workSpaceSize;
  bool allowTensorOpMathConversion;
  ffStream_t stream;     // one stream per handle (the reference creates one per call)
};

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

device_stream_t get_gpu_device_stream();
device_stream_t get_cpu_device_stream();
device_stream_t get_stream_for_device_type(DeviceType);

// RAII stream (reference: lib/kernels/include/kernels/managed_ff_stream.h)
struct ManagedFFStream {
  ManagedFFStream();
  ManagedFFStream(ManagedFFStream const &) = delete;
  ManagedFFStream &operator=(ManagedFFStream const &) = delete;
  ManagedFFStream(ManagedFFStream &&other) noexcept;
  ~ManagedFFStream();
  ffStream_t const &raw_stream() const { return stream; }
 private:
  ffStream_t stream;
};

// RAII handle + workspace (reference: managed_per_device_ff_handle.h,
// src/managed_per_device_ff_handle.cc:7-48)
struct ManagedPerDeviceFFHandle {
  ManagedPerDeviceFFHandle(size_t workSpaceSize, bool allowTensorOpMathConversion);
  ManagedPerDeviceFFHandle(ManagedPerDeviceFFHandle const &) = delete;
  ManagedPerDeviceFFHandle &operator=(ManagedPerDeviceFFHandle const &) = delete;
  ManagedPerDeviceFFHandle(ManagedPerDeviceFFHandle &&other) noexcept;
  ~ManagedPerDeviceFFHandle();
  PerDeviceFFHandle const &raw_handle() const { return handle; }
 private:
  PerDeviceFFHandle handle;
  bool owns;
};
ManagedPerDeviceFFHandle initialize_single_gpu_handle(size_t workSpaceSize,
                                                      bool allowTensorOpMathConversion);
device_handle_t device_handle_t_from_managed_ff_handle(ManagedPerDeviceFFHandle const &);

}  // namespace FlexFlow
