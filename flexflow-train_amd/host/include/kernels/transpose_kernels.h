// Transpose entry points (reference: lib/kernels/include/kernels/transpose_kernels.h:11-19;
// attrs lib/op-attrs/include/op-attrs/ops/transpose_attrs.dtg.toml).
#pragma once
#include "kernels/accessor.h"
#include "kernels/device_stream_t.h"
#include "op-attrs/attrs.h"
#include <vector>

namespace FlexFlow {

namespace Kernels::Transpose {
void forward_kernel(device_stream_t const &stream, TransposeAttrs const &attrs, GenericTensorAccessorR const &input,
                    GenericTensorAccessorW const &output);
// in_grad += out_grad moved back through the inverse permutation
void backward_kernel(device_stream_t const &stream, TransposeAttrs const &attrs, GenericTensorAccessorR const &out_grad,
                     GenericTensorAccessorW const &in_grad);
}  // namespace Kernels::Transpose

}  // namespace FlexFlow
