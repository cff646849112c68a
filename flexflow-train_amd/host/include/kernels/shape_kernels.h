// Transpose, Reshape, Split and Gather entry points (reference:
// lib/kernels/include/kernels/transpose_kernels.h:11-19, reshape_kernels.h:9-15,
// split_kernels.h:9-25, gather_kernels.h:12-30; attrs
// lib/op-attrs/include/op-attrs/ops/transpose_attrs.dtg.toml).
#pragma once
#include "kernels/accessor.h"
#include "kernels/device_stream_t.h"
#include "op-attrs/attrs.h"
#include <vector>

namespace FlexFlow {

struct GatherPerDeviceState {
  PerDeviceFFHandle handle;
  ff_dim_t dim;
};

namespace Kernels::Transpose {
void forward_kernel(device_stream_t const &stream, TransposeAttrs const &attrs, GenericTensorAccessorR const &input,
                    GenericTensorAccessorW const &output);
// in_grad += out_grad moved back through the inverse permutation
void backward_kernel(device_stream_t const &stream, TransposeAttrs const &attrs, GenericTensorAccessorR const &out_grad,
                     GenericTensorAccessorW const &in_grad);
}  // namespace Kernels::Transpose

namespace Kernels::Reshape {
void forward_kernel(device_stream_t const &stream, GenericTensorAccessorR const &input,
                    GenericTensorAccessorW const &output);
// input (gradient) += output (gradient)
void backward_kernel(device_stream_t const &stream, GenericTensorAccessorR const &output,
                     GenericTensorAccessorW const &input);
}  // namespace Kernels::Reshape

namespace Kernels::Split {
void forward_kernel(device_stream_t const &stream, float **out_ptrs, float const *in_ptr, int const *out_blk_sizes,
                    int in_blk_size, int num_blks, int numOutputs);
// in_grad += the output gradients side by side
void backward_kernel(device_stream_t const &stream, float *in_grad_ptr, float const **out_grad_ptr,
                     int const *out_blk_sizes, int in_blk_size, int num_blks, int numOutputs);
}  // namespace Kernels::Split

namespace Kernels::Gather {
std::optional<GatherPerDeviceState> init_kernel(DeviceType device_type, device_handle_t const &handle, ff_dim_t dim);
void forward_kernel(device_stream_t const &stream, std::optional<GatherPerDeviceState> const &per_device_state,
                    GenericTensorAccessorR const &input, GenericTensorAccessorR const &index,
                    GenericTensorAccessorW const &output);
void backward_kernel(device_stream_t const &stream, std::optional<GatherPerDeviceState> const &per_device_state,
                     GenericTensorAccessorR const &output_grad, GenericTensorAccessorR const &index,
                     GenericTensorAccessorW const &input_grad);
}  // namespace Kernels::Gather

}  // namespace FlexFlow
