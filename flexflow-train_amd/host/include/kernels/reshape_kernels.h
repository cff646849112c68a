// Reshape entry points (reference: lib/kernels/include/kernels/reshape_kernels.h:9-15).
#pragma once
#include "kernels/accessor.h"
#include "kernels/device_stream_t.h"
#include "op-attrs/attrs.h"
#include <vector>

namespace FlexFlow {

namespace Kernels::Reshape {
void forward_kernel(device_stream_t const &stream, GenericTensorAccessorR const &input,
                    GenericTensorAccessorW const &output);
// input (gradient) += output (gradient)
void backward_kernel(device_stream_t const &stream, GenericTensorAccessorR const &output,
                     GenericTensorAccessorW const &input);
}  // namespace Kernels::Reshape

}  // namespace FlexFlow
