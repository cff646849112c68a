// Cast entry points (reference: lib/kernels/include/kernels/cast_kernels.h:9-17).
#pragma once
#include "kernels/accessor.h"
#include "kernels/device_stream_t.h"

namespace FlexFlow::Kernels::Cast {

void forward_kernel(device_stream_t const &stream, GenericTensorAccessorR const &input,
                    GenericTensorAccessorW const &output);

// input_grad = cast(output_grad) + input_grad
void backward_kernel(device_stream_t const &stream, GenericTensorAccessorR const &output_grad,
                     GenericTensorAccessorW const &input_grad);

}  // namespace FlexFlow::Kernels::Cast
