// Optimizer update entry points (reference: lib/kernels/include/kernels/
// optimizer_kernels.h:11-36).  Single GPU: the reference's GPU branch calls the
// NCCL launcher, whose all-reduce is the identity on one device, so these go
// straight to the update kernel; num_replicas > 1 sums the gradient replicas
// first like the parameter-server launcher.
#pragma once
#include "kernels/accessor.h"
#include "kernels/device.h"
#include "kernels/device_stream_t.h"

namespace FlexFlow {

void sgd_update_task(device_stream_t const &stream, device_handle_t const &handle, float lr,
                     float momentum, bool nesterov, float weight_decay,
                     GenericTensorAccessorR const &weight_grad, int num_replicas,
                     GenericTensorAccessorW const &weight,
                     std::optional<GenericTensorAccessorW> const &sgd_v);

void adam_update_task(device_stream_t const &stream, device_handle_t const &handle, float alpha_t,
                      float beta1, float beta2, float weight_decay, float epsilon,
                      float const *weight_grad_ptr, size_t size, int num_replicas,
                      float *weight_ptr, float *adam_v_ptr, float *adam_m_ptr);

}  // namespace FlexFlow
