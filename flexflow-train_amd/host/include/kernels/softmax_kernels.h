// Softmax entry points (reference: lib/kernels/include/kernels/softmax_kernels.h:
// 12-32; state softmax_per_device_state.dtg.toml).  The descriptor the reference
// builds from (n, c, h, w) is kept as plain ints: softmax runs over c.
#pragma once
#include "kernels/accessor.h"
#include "kernels/device_stream_t.h"

namespace FlexFlow {

struct SoftmaxPerDeviceState {
  PerDeviceFFHandle handle;
  int n, c, h, w;
  ff_dim_t dim;
  DataType data_type;
};

namespace Kernels::Softmax {

std::optional<SoftmaxPerDeviceState> init_kernel(DeviceType device_type,
                                                 device_handle_t const &handle, ff_dim_t dim,
                                                 int input_n, int input_c, int input_h,
                                                 int input_w);
void forward_kernel(device_stream_t const &stream,
                    std::optional<SoftmaxPerDeviceState> const &per_device_state,
                    float const *input_ptr, float *output_ptr);
// The reference's backward: a device copy (softmax_kernels.cu:68-78).
void backward_kernel(device_stream_t const &stream, float const *output_grad_ptr,
                     float *input_grad_ptr, size_t num_elements);
// extension: accessor overloads (dtype from the shape) and the true gradient
// dx = y * (dy - sum(y * dy)), which needs the forward output.
void forward_kernel(device_stream_t const &stream,
                    std::optional<SoftmaxPerDeviceState> const &per_device_state,
                    GenericTensorAccessorR const &input, GenericTensorAccessorW const &output);
void backward_kernel(device_stream_t const &stream,
                     std::optional<SoftmaxPerDeviceState> const &per_device_state,
                     GenericTensorAccessorR const &output, GenericTensorAccessorR const &output_grad,
                     GenericTensorAccessorW const &input_grad);
void cleanup_kernel(DeviceType device_type,
                    std::optional<SoftmaxPerDeviceState> &per_device_state);

}  // namespace Kernels::Softmax
}  // namespace FlexFlow
