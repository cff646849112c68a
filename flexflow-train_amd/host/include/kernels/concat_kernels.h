// Concat entry points (reference: lib/kernels/include/kernels/concat_kernels.h:9-17).
#pragma once
#include "kernels/accessor.h"
#include "kernels/device_stream_t.h"
#include <vector>

namespace FlexFlow::Kernels::Concat {

void forward_kernel(device_stream_t const &stream, GenericTensorAccessorW const &output,
                    std::vector<GenericTensorAccessorR> const &inputs, ff_dim_t axis);

// input_grads[i] += the slice of output_grad that input i produced
void backward_kernel(device_stream_t const &stream, GenericTensorAccessorR const &output_grad,
                     std::vector<GenericTensorAccessorW> const &input_grads, ff_dim_t axis);

}  // namespace FlexFlow::Kernels::Concat
