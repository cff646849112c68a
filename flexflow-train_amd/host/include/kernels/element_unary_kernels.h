// ElementUnary entry points (reference:
// lib/kernels/include/kernels/element_unary_kernels.h:13-39; state
// element_unary_per_device_state.dtg.toml).
#pragma once
#include "kernels/accessor.h"
#include "kernels/device_stream_t.h"
#include "op-attrs/attrs.h"

namespace FlexFlow {

struct ElementUnaryPerDeviceState {
  TensorShape input_shape, output_shape;
  OperatorType op_type;
};

namespace Kernels::ElementUnary {
std::optional<ElementUnaryPerDeviceState> init_kernel(DeviceType device_type,
                                                      TensorShape const &input_shape,
                                                      TensorShape const &output_shape,
                                                      ElementUnaryAttrs const &attrs);
void forward_kernel(device_stream_t const &stream,
                    std::optional<ElementUnaryPerDeviceState> const &device_state,
                    ElementUnaryAttrs const &attrs, device_handle_t const &handle,
                    GenericTensorAccessorR const &input, GenericTensorAccessorW const &output);
void backward_kernel(device_stream_t const &stream,
                     std::optional<ElementUnaryPerDeviceState> const &device_state,
                     ElementUnaryAttrs const &attrs, device_handle_t const &handle,
                     GenericTensorAccessorR const &output, GenericTensorAccessorR const &output_grad,
                     GenericTensorAccessorR const &input, GenericTensorAccessorW const &input_grad);
void cleanup_kernel(DeviceType device_type,
                    std::optional<ElementUnaryPerDeviceState> &per_device_state);
}  // namespace Kernels::ElementUnary
}  // namespace FlexFlow
