// Linear entry points with the reference's signatures
// (lib/kernels/include/kernels/linear_kernels.h:15-50) and per-device state
// (linear_per_device_state.dtg.toml).
#pragma once
#include "kernels/accessor.h"
#include "kernels/device_stream_t.h"
#include "op-attrs/attrs.h"

namespace FlexFlow {

struct LinearPerDeviceState {
  PerDeviceFFHandle handle;
  // Scratch for the activation-processed output gradient and the bias-gradient
  // partial sums, sized at init from (batch_size, output_num_channels).  The
  // reference keeps a ones-vector here (one_ptr) and cudaMallocs a copy of the
  // output gradient on every backward call (linear_kernels.cc:104-106).
  void *workspace;
  size_t workspace_bytes;
  std::optional<Activation> activation;
  std::optional<RegularizerAttrs> regularizer;
  bool use_bias;
  DataType input_type, weight_type, output_type;
};

std::optional<LinearPerDeviceState> linear_init_kernel(
    DeviceType device_type, device_handle_t const &handle, std::optional<Activation> activation,
    std::optional<RegularizerAttrs> regularizer, bool use_bias, DataType input_type,
    DataType weight_type, DataType output_type, int batch_size, int output_num_channels);

void linear_forward_kernel(device_stream_t const &stream,
                           std::optional<LinearPerDeviceState> const &per_device_state,
                           LinearAttrs const &attrs, GenericTensorAccessorR const &input_accessor,
                           GenericTensorAccessorW const &output_accessor,
                           GenericTensorAccessorR const &projection_accessor,
                           std::optional<GenericTensorAccessorR> const &bias_accessor);

void linear_backward_kernel(device_stream_t const &stream,
                            std::optional<LinearPerDeviceState> const &per_device_state,
                            LinearAttrs const &attrs, GenericTensorAccessorR const &output,
                            GenericTensorAccessorR const &output_grad,
                            GenericTensorAccessorR const &input,
                            GenericTensorAccessorW const &input_grad,
                            GenericTensorAccessorR const &projection,
                            GenericTensorAccessorW const &projection_grad,
                            std::optional<GenericTensorAccessorW> const &bias_grad);

void linear_cleanup_kernel(DeviceType device_type,
                           std::optional<LinearPerDeviceState> &per_device_state);

}  // namespace FlexFlow
