// Gather entry points (reference: lib/kernels/include/kernels/gather_kernels.h:12-30; state
// gather_per_device_state.dtg.toml).
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
