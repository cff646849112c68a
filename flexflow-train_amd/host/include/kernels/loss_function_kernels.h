// Loss-function backward entry points (reference: lib/kernels/include/kernels/
// loss_function_kernels.h:9-45).
#pragma once
#include "kernels/accessor.h"
#include "kernels/device_stream_t.h"

namespace FlexFlow {

void sparse_categorical_crossentropy_loss_backward_kernel(
    device_stream_t const &stream, float *logit_grad_ptr, float const *logit_ptr,
    int const *label_ptr, size_t logit_volume, size_t logit_grad_volume, int num_samples,
    int num_classes, int k, float scale_factor);

void categorical_crossentropy_loss_backward_kernel(device_stream_t const &stream,
                                                   GenericTensorAccessorW const &logit_grad,
                                                   GenericTensorAccessorR const &logit,
                                                   GenericTensorAccessorR const &label,
                                                   float scale_factor);

void mean_squared_error_avg_loss_backward_kernel(device_stream_t const &stream, float *logit_grad_ptr,
                                                 float const *logit_ptr, float const *label_ptr,
                                                 size_t logit_volume, size_t logit_grad_volume,
                                                 float scale_factor);

void identity_loss_backward_kernel(device_stream_t const &stream, float *loss_grad_ptr,
                                   float const *loss_ptr, size_t loss_volume,
                                   size_t loss_grad_volume, float scale_factor);

}  // namespace FlexFlow
