// Split entry points (reference: lib/kernels/include/kernels/split_kernels.h:9-25).
#pragma once
#include "kernels/accessor.h"
#include "kernels/device_stream_t.h"
#include "op-attrs/attrs.h"
#include <vector>

namespace FlexFlow {

namespace Kernels::Split {
void forward_kernel(device_stream_t const &stream, float **out_ptrs, float const *in_ptr, int const *out_blk_sizes,
                    int in_blk_size, int num_blks, int numOutputs);
// in_grad += the output gradients side by side
void backward_kernel(device_stream_t const &stream, float *in_grad_ptr, float const **out_grad_ptr,
                     int const *out_blk_sizes, int in_blk_size, int num_blks, int numOutputs);
}  // namespace Kernels::Split

}  // namespace FlexFlow
