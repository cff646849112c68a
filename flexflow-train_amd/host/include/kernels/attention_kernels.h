// MultiHeadAttention entry points (reference:
// lib/kernels/include/kernels/attention_kernels.h:12-51; state
// mha_per_device_state.dtg.toml).  The float* signatures are the reference's
// (fp32 tensors, a state from the reference's init_kernel); the accessor
// overloads carry the dtype (FLOAT or BF16).  scale / causal are state fields
// with the reference's values (1.0, false) as defaults.  Like cuDNN's calls,
// backward stores the input gradients and adds into the weight gradient.
// Limits: qProjSize == kProjSize == vProjSize; FLOAT: a multiple of 4 up to
// 128; BF16: 64 or 128.
#pragma once
#include "kernels/accessor.h"
#include "kernels/allocation.h"
#include "kernels/device_stream_t.h"

namespace FlexFlow {

struct MHAPerDeviceState {
  PerDeviceFFHandle handle;
  size_t weightSize;        // bytes, like the reference
  size_t reserveSpaceSize;  // bytes
  int num_samples, num_heads, qSize, kSize, vSize, qProjSize, kProjSize, vProjSize, oProjSize;
  int qoSeqLength, kvSeqLength;
  float scale;
  bool causal;
  DataType data_type;
  void *reserveSpace;
  Allocator allocator;
};

namespace Kernels::MultiHeadAttention {

std::optional<MHAPerDeviceState> init_kernel(DeviceType device_type,
                                             device_handle_t const &per_device_ff_handle,
                                             Allocator &allocator, int num_samples, int num_heads,
                                             int qSize, int kSize, int vSize, int qProjSize,
                                             int kProjSize, int vProjSize, int oProjSize,
                                             int qoSeqLength, int kvSeqLength, bool add_bias_kv);
// extension: dtype, softmax scale and causal mask
std::optional<MHAPerDeviceState> init_kernel(DeviceType device_type,
                                             device_handle_t const &per_device_ff_handle,
                                             Allocator &allocator, int num_samples, int num_heads,
                                             int qSize, int kSize, int vSize, int qProjSize,
                                             int kProjSize, int vProjSize, int oProjSize,
                                             int qoSeqLength, int kvSeqLength, bool add_bias_kv,
                                             DataType data_type, float scale, bool causal);

void forward_kernel(device_stream_t const &stream,
                    std::optional<MHAPerDeviceState> const &device_state, float const *query_ptr,
                    float const *key_ptr, float const *value_ptr, float const *weight_ptr,
                    float *output_ptr);
void forward_kernel(device_stream_t const &stream,
                    std::optional<MHAPerDeviceState> const &device_state,
                    GenericTensorAccessorR const &query, GenericTensorAccessorR const &key,
                    GenericTensorAccessorR const &value, GenericTensorAccessorR const &weight,
                    GenericTensorAccessorW const &output);

void backward_kernel(device_stream_t const &stream,
                     std::optional<MHAPerDeviceState> const &device_state, float const *query_ptr,
                     float *query_grad_ptr, float const *key_ptr, float *key_grad_ptr,
                     float const *value_ptr, float *value_grad_ptr, float const *weight_ptr,
                     float *weight_grad_ptr, float const *output_grad_ptr);
// key_grad / value_grad may be nullopt when key / value alias query.
void backward_kernel(device_stream_t const &stream,
                     std::optional<MHAPerDeviceState> const &device_state,
                     GenericTensorAccessorR const &query, GenericTensorAccessorW const &query_grad,
                     GenericTensorAccessorR const &key,
                     std::optional<GenericTensorAccessorW> const &key_grad,
                     GenericTensorAccessorR const &value,
                     std::optional<GenericTensorAccessorW> const &value_grad,
                     GenericTensorAccessorR const &weight, GenericTensorAccessorW const &weight_grad,
                     GenericTensorAccessorR const &output_grad);

void cleanup_kernel(DeviceType device_type, Allocator &allocator,
                    std::optional<MHAPerDeviceState> const &device_state);

}  // namespace Kernels::MultiHeadAttention
}  // namespace FlexFlow
