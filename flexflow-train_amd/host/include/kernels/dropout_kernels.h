// Dropout entry points (reference: lib/kernels/include/kernels/dropout_kernels.h:
// 12-34; state dropout_per_device_state.dtg.toml).  No reserve space or generator
// state is kept: the mask is a function of (seed, element index).
#pragma once
#include "kernels/accessor.h"
#include "kernels/allocation.h"
#include "kernels/device_stream_t.h"

namespace FlexFlow {

struct DropoutPerDeviceState {
  PerDeviceFFHandle handle;
  float rate;
  unsigned long long seed;
  TensorShape output_shape;
};

namespace Kernels::Dropout {

std::optional<DropoutPerDeviceState> init_kernel(DeviceType device_type,
                                                 device_handle_t const &handle, float rate,
                                                 unsigned long long seed,
                                                 TensorShape const &output_shape,
                                                 Allocator &allocator);
void forward_kernel(device_stream_t const &stream,
                    std::optional<DropoutPerDeviceState> const &per_device_state,
                    float const *input_ptr, float *output_ptr);
void backward_kernel(device_stream_t const &stream,
                     std::optional<DropoutPerDeviceState> const &per_device_state,
                     float const *output_grad_ptr, float *input_grad_ptr);
// extension: dtype taken from the accessor
void forward_kernel(device_stream_t const &stream,
                    std::optional<DropoutPerDeviceState> const &per_device_state,
                    GenericTensorAccessorR const &input, GenericTensorAccessorW const &output);
void backward_kernel(device_stream_t const &stream,
                     std::optional<DropoutPerDeviceState> const &per_device_state,
                     GenericTensorAccessorR const &output_grad,
                     GenericTensorAccessorW const &input_grad);
void cleanup_kernel(DeviceType device_type, Allocator &allocator,
                    std::optional<DropoutPerDeviceState> &per_device_state);

}  // namespace Kernels::Dropout
}  // namespace FlexFlow
