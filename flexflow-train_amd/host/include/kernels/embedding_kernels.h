// Embedding entry points (reference: lib/kernels/include/kernels/
// embedding_kernels.h:10-30).  The reference's task passes the tensors' RANK
// as in_dim/out_dim (lib/task-spec/src/task-spec/ops/impl/embedding.cc:30-31);
// sizes are therefore derived from the accessor shapes and those two
// arguments are ignored.
#pragma once
#include "kernels/accessor.h"
#include "kernels/device_stream_t.h"
#include "op-attrs/attrs.h"

namespace FlexFlow::Kernels::Embedding {

void forward_kernel(device_stream_t const &stream, GenericTensorAccessorR const &input,
                    GenericTensorAccessorW const &output, GenericTensorAccessorR const &weight,
                    DataType input_data_type, DataType output_data_type,
                    std::optional<AggregateOp> aggr, num_tensor_dims_t in_dim,
                    num_tensor_dims_t out_dim, int batch_size);

// `output` carries the output GRADIENT; weight_grad is fp32 and accumulated into.
void backward_kernel(device_stream_t const &stream, GenericTensorAccessorR const &output,
                     GenericTensorAccessorR const &input, GenericTensorAccessorW const &weight_grad,
                     DataType output_data_type, DataType input_data_type,
                     std::optional<AggregateOp> aggr, num_tensor_dims_t in_dim,
                     num_tensor_dims_t out_dim, int batch_size);

}  // namespace FlexFlow::Kernels::Embedding
