// ElementBinary entry points (reference:
// lib/kernels/include/kernels/element_binary_kernels.h:16-51; state
// element_binary_per_device_state.dtg.toml).
#pragma once
#include "kernels/accessor.h"
#include "kernels/device_stream_t.h"
#include "op-attrs/attrs.h"

namespace FlexFlow {

struct ElementBinaryPerDeviceState {
  PerDeviceFFHandle handle;
  OperatorType op_type;
  bool should_broadcast_lhs, should_broadcast_rhs;
  TensorShape lhs_shape, rhs_shape, output_shape;
};

namespace Kernels::ElementBinary {
std::optional<ElementBinaryPerDeviceState> init_kernel(
    DeviceType device_type, device_handle_t const &handle, OperatorType op_type,
    bool should_broadcast_lhs, bool should_broadcast_rhs, TensorShape const &lhs_shape,
    TensorShape const &rhs_shape, TensorShape const &output_shape);
// fp32 pointers (the reference's signatures); gradients accumulate (beta = 1).
void forward_kernel(device_stream_t const &stream,
                    std::optional<ElementBinaryPerDeviceState> const &per_device_state,
                    float const *lhs_ptr, float const *rhs_ptr, float *out_ptr,
                    OperatorType op_type, bool broadcast_inputLHS, device_handle_t const &handle);
void backward_kernel(device_stream_t const &stream,
                     std::optional<ElementBinaryPerDeviceState> const &per_device_state,
                     float const *out_grad_ptr, float const *lhs_ptr, float const *rhs_ptr,
                     float *lhs_grad_ptr, float *rhs_grad_ptr, OperatorType op_type,
                     bool broadcast_inputLHS, bool broadcast_inputRHS,
                     device_handle_t const &handle);
// extension: dtype from the accessors
void forward_kernel(device_stream_t const &stream,
                    std::optional<ElementBinaryPerDeviceState> const &per_device_state,
                    GenericTensorAccessorR const &lhs, GenericTensorAccessorR const &rhs,
                    GenericTensorAccessorW const &out);
void backward_kernel(device_stream_t const &stream,
                     std::optional<ElementBinaryPerDeviceState> const &per_device_state,
                     GenericTensorAccessorR const &out_grad, GenericTensorAccessorR const &lhs,
                     GenericTensorAccessorR const &rhs, GenericTensorAccessorW const &lhs_grad,
                     GenericTensorAccessorW const &rhs_grad);
void cleanup_kernel(DeviceType device_type,
                    std::optional<ElementBinaryPerDeviceState> const &per_device_state);
}  // namespace Kernels::ElementBinary
}  // namespace FlexFlow
