// LayerNorm entry points (reference: lib/kernels/include/kernels/
// layer_norm_kernels.h:12-41; state layer_norm_per_device_state.dtg.toml).
#pragma once
#include "kernels/accessor.h"
#include "kernels/allocation.h"
#include "kernels/device_stream_t.h"

namespace FlexFlow {

struct LayerNormPerDeviceState {
  PerDeviceFFHandle handle;
  bool elementwise_affine;
  int64_t effective_num_elements;  // N, the normalised extent
  int64_t effective_batch_size;    // M
  float eps;
  float *mean, *rstd;              // [M] fp32, written by forward
  void *workspace;                 // partial dgamma/dbeta sums (replaces ds, db, scale, bias)
  size_t workspace_bytes;
  DataType data_type;
};

namespace Kernels::LayerNorm {

std::optional<LayerNormPerDeviceState> init_kernel(DeviceType device_type,
                                                   device_handle_t const &handle,
                                                   Allocator &allocator, bool elementwise_affine,
                                                   int64_t effective_batch_size,
                                                   int64_t effective_num_elements, float eps);

void forward_kernel(device_stream_t const &stream,
                    std::optional<LayerNormPerDeviceState> const &per_device_state,
                    GenericTensorAccessorR const &input, GenericTensorAccessorW const &output,
                    GenericTensorAccessorW const &gamma, GenericTensorAccessorW const &beta);

// Also writes input_grad (the reference defines that kernel but never launches
// it, layer_norm_kernels.cu:163-181,354-410).
void backward_kernel(device_stream_t const &stream,
                     std::optional<LayerNormPerDeviceState> const &per_device_state,
                     GenericTensorAccessorR const &output_grad, GenericTensorAccessorR const &input,
                     GenericTensorAccessorW const &input_grad, GenericTensorAccessorR const &gamma,
                     GenericTensorAccessorW const &gamma_grad,
                     GenericTensorAccessorW const &beta_grad);

void cleanup_kernel(DeviceType device_type,
                    std::optional<LayerNormPerDeviceState> const &per_device_state);

}  // namespace Kernels::LayerNorm
}  // namespace FlexFlow
