#pragma once
#include "kernels/device_handle_t.h"
#include "kernels/ff_handle.h"

namespace FlexFlow {

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
