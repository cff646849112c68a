// Fused passes behind the encoder-layer entry points.  Each one produces
// exactly the bits the corresponding sequence of separate operator kernels
// would (intermediate values are rounded to the storage type where the
// separate ops would have stored them), and saves the intermediate tensor's
// trip through HBM.  Internal: the C ABI exposes only the separate ops and the
// layer entry points.
#pragma once
#include "ffk_common.h"

namespace ffk {

// True when the operands allow the vector kernels below (whole 16-byte
// chunks, aligned pointers, offset a multiple of 4).
bool dropout_fusable(int dtype, void const *x, void const *aux, void const *y,
                     int64_t n, uint64_t offset);

// y = residual + dropout(x)
int dropout_add_residual(hipStream_t st, int dtype, void const *x,
                         void const *residual, void *y, int64_t n, float rate,
                         uint64_t seed, uint64_t offset);

// dx = dropout_backward(dy) * GELU'(gelu_input)
int dropout_backward_gelu_backward(hipStream_t st, int dtype, void const *dy,
                                   void const *gelu_input, void *dx, int64_t n,
                                   float rate, uint64_t seed, uint64_t offset);

// y = dropout(GELU(x)) with GELU's output rounded to the storage type first
int gelu_dropout_forward(hipStream_t st, int dtype, void const *x, void *y,
                         int64_t n, float rate, uint64_t seed, uint64_t offset);

// output = input . weight^T + bias (stored: backward reads it);
// dropped = dropout(GELU(output)), written by the GEMM while it stores its
// tile.  FFK_ERR_UNSUPPORTED (no error message) when the shape does not run on
// the pipelined bf16 GEMM tiles.
int linear_gelu_dropout_forward(hipStream_t st, int dtype, void const *input, void *output,
                                void *dropped, void const *weight, void const *bias, int64_t batch,
                                int64_t in_dim, int64_t out_dim, float rate, uint64_t seed,
                                uint64_t offset);

// output = residual + dropout(input . weight^T + bias); Linear's own output
// is not stored.  FFK_ERR_UNSUPPORTED as above.
int linear_dropout_add_forward(hipStream_t st, int dtype, void const *input, void const *residual,
                               void *output, void const *weight, void const *bias, int64_t batch,
                               int64_t in_dim, int64_t out_dim, float rate, uint64_t seed,
                               uint64_t offset);

// Linear backward (no activation) whose input gradient is
// dropout_backward(output_grad . weight) * GELU'(gelu_input): the gradient of
// Linear's input never reaches memory on its own.  weight_grad / bias_grad as
// ffk_linear_backward.  FFK_ERR_UNSUPPORTED as above, before any launch.
int linear_backward_dropout_gelu(hipStream_t st, int dtype, void const *output_grad, void const *input,
                                 void const *gelu_input, void *input_grad, void const *weight,
                                 void *weight_grad, void *bias_grad, int64_t batch, int64_t in_dim,
                                 int64_t out_dim, void *workspace, size_t workspace_bytes,
                                 int accumulate, float rate, uint64_t seed, uint64_t offset,
                                 // optional: input_grad_colsum [in_dim] (+)= column sums of input_grad as
                                 // stored (the bias gradient of the Linear in front of the GELU), the bits
                                 // of the separate column-sum kernel; colsum_partials: fp32 scratch of
                                 // colsum_partials_elems(batch, in_dim) that nothing else uses until the
                                 // sums are complete
                                 void *input_grad_colsum = nullptr, float *colsum_partials = nullptr,
                                 bool colsum_accumulate = false);

// summed = residual + dropout(in); y = LayerNorm(summed), statistics kept as the separate
// LayerNorm would.  Returns FFK_ERR_UNSUPPORTED (without setting an error
// message) when the row length or the alignment has no vector kernel.
int dropout_add_layer_norm_forward(hipStream_t st, int dtype, void const *in, void const *residual,
                                   void *summed, void *y, void const *gamma, void const *beta,
                                   float *mean, float *rstd, int64_t M, int64_t N, float eps,
                                   float rate, uint64_t seed, uint64_t offset);

// dx = residual + LayerNorm_backward(dy) (dgamma/dbeta as the separate op);
// FFK_ERR_UNSUPPORTED when the row length has no vector kernel.
int layer_norm_backward_add_residual(hipStream_t st, int dtype, void const *dy,
                                     void const *x, float const *mean,
                                     float const *rstd, void const *gamma,
                                     void const *residual, void *dx,
                                     void *dgamma, void *dbeta, int64_t M,
                                     int64_t N, void *workspace,
                                     size_t workspace_bytes,
                                     // optional: dropped = dropout_backward(dx as stored)
                                     void *dropped = nullptr, float rate = 0.0f,
                                     uint64_t seed = 0, uint64_t offset = 0,
                                     // dgamma / dbeta are added to instead of stored
                                     bool acc_params = false,
                                     // the gradient is rounded to the storage type before residual
                                     // is added (what a separate add of the stored gradient gives);
                                     // false: the sum is rounded once (what adding the gradient
                                     // into a copy of residual gives)
                                     bool round_first = true);

}  // namespace ffk
