/*
 * ffk.h -- C ABI of the gfx950 (MI355X) operator-kernel library libffk.so.
 *
 * Every function is what the reference's `Kernels::<Op>::gpu_*_kernel`
 * (lib/kernels/include/kernels/<op>_kernels_gpu.h) does for one operator on one
 * device, with the C++ value types flattened to plain pointers, sizes and
 * enum ordinals so it can be bound from any host language.
 *
 * Conventions
 *  - All tensor pointers are DEVICE pointers to dense row-major data (FF dim
 *    order: dim 0 outermost, last dim contiguous; reference
 *    lib/kernels/src/kernels/accessor.cc:15-33).
 *  - Every call is asynchronous on `stream` (a hipStream_t passed as void*)
 *    and never synchronises (reference: only profiling_wrapper syncs,
 *    lib/kernels/include/kernels/profiling.h:78-106).
 *  - Return value: FFK_OK (0) or an FFK_ERR_* code; ffk_last_error() returns
 *    the calling thread's message. No C++ exception crosses the boundary.
 *  - `accumulate` != 0 means the gradient output is added to (the reference
 *    GPU path's beta = 1), 0 means it is overwritten.
 *  - dtype arguments use the ordinals of the reference's DataType enum
 *    (lib/op-attrs/include/op-attrs/datatype.dtg.toml:11-27) plus BF16.
 *  - There is no CPU fallback inside this library.
 */
#ifndef FFK_H
#define FFK_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *ffk_stream_t; /* hipStream_t; NULL = the null stream */
typedef void *ffk_event_t;  /* hipEvent_t */

enum {
  FFK_OK = 0,
  FFK_ERR_INVALID = 1,     /* precondition on shapes/dtypes/pointers failed */
  FFK_ERR_HIP = 2,         /* a HIP runtime call failed */
  FFK_ERR_UNSUPPORTED = 3, /* combination not implemented */
  FFK_ERR_WORKSPACE = 4    /* caller-provided workspace too small */
};

/* DataType ordinals (datatype.dtg.toml:11-27); BF16 is appended. */
enum {
  FFK_BOOL = 0,
  FFK_INT32 = 1,
  FFK_INT64 = 2,
  FFK_HALF = 3,
  FFK_FLOAT = 4,
  FFK_DOUBLE = 5,
  FFK_BF16 = 6
};

/* Activation ordinals (lib/op-attrs/include/op-attrs/activation.dtg.toml). */
enum {
  FFK_ACT_NONE = -1,
  FFK_ACT_RELU = 0,
  FFK_ACT_SIGMOID = 1,
  FFK_ACT_TANH = 2,
  FFK_ACT_GELU = 3
};

/* OperatorType ordinals used by the element-wise kernels
 * (lib/op-attrs/include/op-attrs/operator_type.dtg.toml:12-94). */
enum {
  FFK_OP_SCALAR_MULTIPLY = 8,
  FFK_OP_SCALAR_ADD = 9,
  FFK_OP_SCALAR_TRUE_DIV = 11,
  FFK_OP_SCALAR_SUB = 12,
  FFK_OP_RELU = 13,
  FFK_OP_IDENTITY = 14,
  FFK_OP_SIGMOID = 15,
  FFK_OP_TANH = 16,
  FFK_OP_ELU = 17,
  FFK_OP_EW_ADD = 28,
  FFK_OP_EW_MUL = 29,
  FFK_OP_EW_SUB = 35,
  FFK_OP_EW_DIV = 36,
  FFK_OP_EW_MAX = 40,
  FFK_OP_EW_MIN = 41,
  FFK_OP_EXP = 56,
  FFK_OP_SIN = 61,
  FFK_OP_COS = 62,
  FFK_OP_GELU = 67,
  FFK_OP_RSQRT = 70,
  FFK_OP_POW = 71,
  /* not a reference ordinal: GELU whose backward is the literal formula of
   * element_unary_kernels.cu:226-231 (0.5 erfc(-x/sqrt2) - 0.5/sqrt2 x exp(-x^2/2))
   * instead of the true derivative Phi(x) + x phi(x) */
  FFK_OP_GELU_REFERENCE_GRAD = 1067
};

/* AggregateOp (lib/op-attrs/include/op-attrs/aggregate_op.dtg.toml). */
enum { FFK_AGGR_NONE = -1, FFK_AGGR_SUM = 0, FFK_AGGR_AVG = 1 };

/* ------------------------------------------------------------------------ */
/* Runtime shim: the only way host C++ reaches HIP (no hip headers above it).
 * Replaces the cudaMalloc/cudaMemcpy/cudaStreamCreate/cudaEvent* calls of
 * lib/kernels/src/kernels/local_cuda_allocator.cc, accessor.cc:45-74,
 * managed_ff_stream.cc and include/kernels/profiling.h:78-106.              */
/* ------------------------------------------------------------------------ */
char const *ffk_last_error(void);
int ffk_device_count(int *count);
int ffk_set_device(int device);
int ffk_malloc(void **ptr, size_t bytes);
int ffk_free(void *ptr);
int ffk_host_malloc(void **ptr, size_t bytes); /* pinned host memory */
int ffk_host_free(void *ptr);
enum { FFK_H2D = 1, FFK_D2H = 2, FFK_D2D = 3 };
int ffk_memcpy(void *dst, void const *src, size_t bytes, int kind,
               ffk_stream_t stream); /* blocking when stream == NULL */
int ffk_fill_zero(void *ptr, size_t bytes, ffk_stream_t stream);
int ffk_stream_create(ffk_stream_t *stream);
int ffk_stream_destroy(ffk_stream_t stream);
int ffk_stream_synchronize(ffk_stream_t stream);
int ffk_event_create(ffk_event_t *ev);
int ffk_event_destroy(ffk_event_t ev);
int ffk_event_record(ffk_event_t ev, ffk_stream_t stream);
int ffk_event_synchronize(ffk_event_t ev);
int ffk_event_elapsed_ms(ffk_event_t start, ffk_event_t stop, float *ms);

/* Measurement aid; no counterpart in the reference.  One launch in which
 * every SIMD of the chip issues `iterations` x 16 bf16 32x32x16 matrix
 * instructions back to back from registers (no memory traffic): timed by the
 * caller, *flops / time is the matrix rate this card sustains, the ceiling a
 * GEMM kernel here can approach (the vendor's 2.5 PFLOP/s assumes a clock the
 * chip does not hold under that load).  out: scratch of at least 256 KiB
 * (one float per lane, so the work cannot be dropped).                      */
int ffk_probe_mfma_bf16(ffk_stream_t stream, int iterations, uint32_t seed,
                        float *out, size_t out_bytes, double *flops);

/* Process-wide switches for tuning runs and tests; no counterpart in the
 * reference.  All start at 0 and change through ffk_set_option only: the
 * library never reads the environment.
 *   FFK_OPTION_GEMM_VARIANT: 0 = the dispatch heuristic;
 *     128 / 256 force that pipelined bf16 tile (eight waves), 264 the 256 tile
 *     with one wave per SIMD, 1 the register-staged kernel.
 *   FFK_OPTION_LAYER_UNFUSED: != 0 makes the encoder-layer
 *     entry points (and a step-driver instance created while it is set) run
 *     one kernel per operator.
 *   FFK_OPTION_ATTENTION_VARIANT: which of the two tuned bf16 forward
 *     kernels runs: 0 = 64 query rows per wavefront from 1024 keys on, 32
 *     below; 1 = 32 rows at every size; 2 = 64 rows at every size.          */
enum {
  FFK_OPTION_GEMM_VARIANT = 0,
  FFK_OPTION_LAYER_UNFUSED = 1,
  FFK_OPTION_ATTENTION_VARIANT = 2,
  FFK_OPTION_COUNT = 3
};
int ffk_set_option(int which, int value);
int ffk_get_option(int which, int *value);

/* ------------------------------------------------------------------------ */
/* Linear -- replaces Kernels::Linear::gpu_forward_kernel / gpu_backward_kernel
 * (lib/kernels/include/kernels/linear_kernels_gpu.h:22-43; CUDA body
 * lib/kernels/src/cuda/ops/linear_kernels.cu:121-341) and computes what
 * linear_cpu_forward_kernel / linear_cpu_backward_kernel do
 * (lib/kernels/src/kernels/linear_kernels_cpu.cc:12-94).
 *   input [batch,in], weight [out,in] (lib/op-attrs/src/op-attrs/ops/linear.cc:43-55),
 *   bias [out] or NULL, output [batch,out].  dtype: FFK_FLOAT or FFK_BF16
 *   (bf16 operands, fp32 accumulate, one rounding at the store).
 * forward:  output = act(input . weight^T + bias)
 * backward: g = act'(output) * output_grad; input_grad (+)= g . weight;
 *           weight_grad (+)= g^T . input; bias_grad (+)= sum_batch g.
 *   relu_grad_mode selects the activation gradient for RELU:
 *     0 = g = output_grad * [output > 0]  (reference GPU, cuda_helper.cu:60-64)
 *     1 = g = [output_grad > 0] ? 1 : 0   (reference CPU, linear_kernels_cpu.cc:46-52,65-71)
 *   Any of input_grad / weight_grad / bias_grad may be NULL (skipped).
 *   accumulate is a bit mask of FFK_ACC_INPUT / FFK_ACC_WEIGHT / FFK_ACC_BIAS
 *   (FFK_ACC_ALL = the reference GPU path, beta = 1 on all three products,
 *   linear_kernels.cu:262,311,334; 0 = the reference CPU path, which
 *   overwrites, linear_kernels_cpu.cc:80-93).
 *   workspace: device scratch of ffk_linear_backward_workspace_bytes(...)
 *   bytes (holds g when there is an activation, and the partial column sums
 *   of the bias gradient); may be NULL when that size is 0.                  */
/* ------------------------------------------------------------------------ */
int ffk_linear_forward(ffk_stream_t stream, int dtype, int activation,
                       void const *input, void *output, void const *weight,
                       void const *bias, int64_t batch, int64_t in_dim,
                       int64_t out_dim);
enum { FFK_ACC_INPUT = 1, FFK_ACC_WEIGHT = 2, FFK_ACC_BIAS = 4, FFK_ACC_ALL = 7 };
size_t ffk_linear_backward_workspace_bytes(int dtype, int activation,
                                           int use_bias, int64_t batch,
                                           int64_t out_dim);
int ffk_linear_backward(ffk_stream_t stream, int dtype, int activation,
                        int relu_grad_mode, void const *output,
                        void const *output_grad, void const *input,
                        void *input_grad, void const *weight, void *weight_grad,
                        void *bias_grad, int64_t batch, int64_t in_dim,
                        int64_t out_dim, void *workspace,
                        size_t workspace_bytes, int accumulate);

/* The L2 regulariser's term of Linear's weight gradient: weight_grad = 1 *
 * weight_grad + lambda * weight over `elems` elements, what the reference does
 * with one cublasSgeam behind the weight-gradient GEMM of every backward call
 * (lib/kernels/src/cuda/ops/linear_kernels.cu:269-290).  FLOAT or BF16 (fp32
 * arithmetic, one rounding at the store).  The reference asserts on any other
 * regulariser (L1); callers do the same.                                      */
int ffk_linear_l2_regularizer_grad(ffk_stream_t stream, int dtype,
                                   void const *weight, void *weight_grad,
                                   int64_t elems, float lambda);


/* General GEMM behind Linear and the attention projections:
 *   C[M,N] (+)= op(A) . op(B)   with fp32 accumulation.
 *   trans_a == 0: A is [M,K] row-major; 1: A is [K,M] row-major.
 *   trans_b == 0: B is [K,N] row-major; 1: B is [N,K] row-major.
 * Replaces the cublasGemmEx calls of linear_kernels.cu:143,249,321.          */
int ffk_gemm(ffk_stream_t stream, int dtype, int trans_a, int trans_b,
             int64_t M, int64_t N, int64_t K, void const *A, void const *B,
             void *C, int accumulate);

/* Which kernel ffk_gemm / ffk_linear_forward would launch for a dense problem of
 * this data type, kind, shape and epilogue (bias, FFK_ACT_*), as the kernel's
 * template instance, e.g. "gemm_bf16_pipe_kernel<256,256,128,128,64,2,1,false,
 * true,0,false>".  Nothing is launched and no device is touched: the dispatch
 * runs with a name sink in place of the launch.  For reports that must name
 * the kernel they measured; no counterpart in the reference.                  */
int ffk_gemm_kernel_name(int dtype, int trans_a, int trans_b, int64_t M,
                         int64_t N, int64_t K, int has_bias, int activation,
                         char *name, size_t name_bytes);

/* ------------------------------------------------------------------------ */
/* ElementUnary -- Kernels::ElementUnary::gpu_forward_kernel/gpu_backward_kernel
 * (element_unary_kernels_gpu.h:16-30; lib/kernels/src/cuda/ops/
 * element_unary_kernels.cu:104-250,255-380).  `scalar` is used by the
 * SCALAR_* / POW ops and as the ELU coefficient.
 * backward: reference semantics per op (`+=` for most ops, `=` for GELU, POW,
 * RSQRT) when accumulate == -1; 0/1 force overwrite/accumulate uniformly.    */
/* ------------------------------------------------------------------------ */
int ffk_element_unary_forward(ffk_stream_t stream, int dtype, int op_type,
                              float scalar, void const *input, void *output,
                              int64_t num_elements);
int ffk_element_unary_backward(ffk_stream_t stream, int dtype, int op_type,
                               float scalar, void const *output,
                               void const *output_grad, void const *input,
                               void *input_grad, int64_t num_elements,
                               int accumulate);

/* ------------------------------------------------------------------------ */
/* ElementBinary -- Kernels::ElementBinary::gpu_forward_kernel/gpu_backward_kernel
 * (element_binary_kernels_gpu.h:18-37; lib/kernels/src/cuda/ops/
 * element_binary_kernels.cu:27-81,150-427).  ops: EW_ADD/SUB/MUL/DIV/MAX/MIN.
 * lhs_elems / rhs_elems: element counts of the operands; an operand with fewer
 * elements than the output is broadcast as a trailing-dims tensor (index
 * i % operand_elems), which covers the bias-style broadcast the reference
 * builds with cudnnOpTensor (element_binary_kernels.cu:171-234).             */
/* ------------------------------------------------------------------------ */
int ffk_element_binary_forward(ffk_stream_t stream, int dtype, int op_type,
                               void const *lhs, void const *rhs, void *out,
                               int64_t out_elems, int64_t lhs_elems,
                               int64_t rhs_elems);
int ffk_element_binary_backward(ffk_stream_t stream, int dtype, int op_type,
                                void const *out_grad, void const *lhs,
                                void const *rhs, void *lhs_grad, void *rhs_grad,
                                int64_t out_elems, int accumulate);
/* The backward when an operand was broadcast (the reference's broadcast_inputLHS /
 * broadcast_inputRHS branches, element_binary_kernels.cu:268-396: EW_ADD, EW_SUB,
 * EW_MUL; other ops answer FFK_ERR_UNSUPPORTED).  An operand with out_elems
 * elements gets its element-wise gradient; one with fewer gets the sum over the
 * output elements it was broadcast to (index i % operand_elems), added up in a
 * fixed order in fp32.  lhs_grad / rhs_grad may be NULL (that gradient is not
 * computed, as in the reference); accumulate != 0 adds into them (the reference's
 * beta = 1), 0 stores.  EW_MUL reads the other operand of each gradient.      */
int ffk_element_binary_backward_broadcast(ffk_stream_t stream, int dtype, int op_type,
                                          void const *out_grad, void const *lhs,
                                          void const *rhs, void *lhs_grad, void *rhs_grad,
                                          int64_t out_elems, int64_t lhs_elems,
                                          int64_t rhs_elems, int accumulate);

/* ------------------------------------------------------------------------ */
/* LayerNorm -- Kernels::LayerNorm::gpu_forward_kernel / gpu_backward_kernel
 * (layer_norm_kernels_gpu.h:19-33; lib/kernels/src/cuda/ops/
 * layer_norm_kernels.cu:69-181,328-410).  X,Y [M,N]; gamma,beta [N] (NULL =
 * no affine); mean,rstd [M] fp32 written by forward and read by backward
 * (LayerNormPerDeviceState.mean/.rstd).  backward also writes dX -- the
 * formula of LayerNormBackwardCUDAKenrel (layer_norm_kernels.cu:163-181)
 * which the reference defines but never launches.
 * workspace: ffk_layer_norm_backward_workspace_bytes(M, N) bytes (partial
 * column sums for dgamma/dbeta).  accumulate_input_grad is a bit mask:
 * FFK_LN_ACC_INPUT adds into input_grad, FFK_LN_ACC_PARAMS adds into
 * gamma_grad / beta_grad (0: both are stored).                               */
/* ------------------------------------------------------------------------ */
int ffk_layer_norm_forward(ffk_stream_t stream, int dtype, void const *input,
                           void *output, void const *gamma, void const *beta,
                           float *mean, float *rstd, int64_t M, int64_t N,
                           float eps);
enum { FFK_LN_ACC_INPUT = 1, FFK_LN_ACC_PARAMS = 2 };
size_t ffk_layer_norm_backward_workspace_bytes(int64_t M, int64_t N);
int ffk_layer_norm_backward(ffk_stream_t stream, int dtype,
                            void const *output_grad, void const *input,
                            float const *mean, float const *rstd,
                            void const *gamma, void *input_grad,
                            void *gamma_grad, void *beta_grad, int64_t M,
                            int64_t N, void *workspace, size_t workspace_bytes,
                            int accumulate_input_grad);

/* ffk_layer_norm_backward for callers that cannot allocate device memory or
 * bring a workspace: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  It has no counterpart in the reference
 * (whose LayerNorm state allocates its buffers at init,
 * layer_norm_kernels.cu:292-325).  Same arguments and results as
 * ffk_layer_norm_backward without the workspace pair: the partial column sums
 * live in an array of FFK_LAYER_NORM_STATIC_SCRATCH_BYTES that every device
 * the library runs on holds until the process ends.  The call allocates and
 * frees nothing.  Rows longer than FFK_LAYER_NORM_STATIC_MAX_N elements are
 * refused with FFK_ERR_WORKSPACE.  When the array holds fewer partial rows
 * than ffk_layer_norm_backward would use (N above 2048), fewer workgroups
 * walk the rows: input_grad has the same bits, gamma_grad / beta_grad are the
 * same sums taken in a different order.  All calls on one device share the
 * array: calls that overlap on one device (two streams, two threads) race;
 * calls on one stream do not.  Inside ffk_column_reductions_begin/_end its
 * column reduction is launched at once, not collected.                       */
#define FFK_LAYER_NORM_STATIC_SCRATCH_BYTES (8u << 20)
#define FFK_LAYER_NORM_STATIC_MAX_N 16384
int ffk_layer_norm_backward_static(ffk_stream_t stream, int dtype,
                                   void const *output_grad, void const *input,
                                   float const *mean, float const *rstd,
                                   void const *gamma, void *input_grad,
                                   void *gamma_grad, void *beta_grad, int64_t M,
                                   int64_t N, int accumulate_input_grad);

/* ------------------------------------------------------------------------ */
/* Softmax -- Kernels::Softmax::gpu_forward_kernel / gpu_backward_kernel
 * (softmax_kernels_gpu.h:18-26; lib/kernels/src/cuda/ops/softmax_kernels.cu:
 * 45-78).  The tensor is viewed as [outer, dim_size, inner]; softmax is taken
 * over dim_size (cudnnSoftmaxForward ACCURATE/MODE_CHANNEL is outer = n,
 * dim_size = c, inner = h*w).
 * ffk_softmax_backward_copy is the reference's backward (a device copy,
 * softmax_kernels.cu:68-78); ffk_softmax_backward is the true gradient
 * dx = y * (dy - sum(y * dy)).                                               */
/* ------------------------------------------------------------------------ */
int ffk_softmax_forward(ffk_stream_t stream, int dtype, void const *input,
                        void *output, int64_t outer, int64_t dim_size,
                        int64_t inner);
int ffk_softmax_backward_copy(ffk_stream_t stream, int dtype,
                              void const *output_grad, void *input_grad,
                              size_t num_elements);
int ffk_softmax_backward(ffk_stream_t stream, int dtype, void const *output,
                         void const *output_grad, void *input_grad,
                         int64_t outer, int64_t dim_size, int64_t inner);

/* ------------------------------------------------------------------------ */
/* Dropout -- Kernels::Dropout::gpu_forward_kernel / gpu_backward_kernel
 * (dropout_kernels_gpu.h:18-26; lib/kernels/src/cuda/ops/dropout_kernels.cu:
 * 60-95, where the mask comes from cuDNN's opaque generator).  Here the mask
 * is a pure function of (seed, offset + element index): Philox4x32-10 with
 * key = (seed low 32, seed high 32), counter = (e/8 low, e/8 high, 0, 0) for
 * e = offset + i; element e owns 16 of the block's 128 bits -- half (e%8)%2
 * (0 = low) of word (e%8)/2 -- and is kept iff they are >= ceil(rate * 2^16);
 * kept elements are scaled by 1/(1-rate).  No mask is stored: backward
 * regenerates it.                                                            */
/* ------------------------------------------------------------------------ */
int ffk_dropout_forward(ffk_stream_t stream, int dtype, void const *input,
                        void *output, int64_t num_elements, float rate,
                        uint64_t seed, uint64_t offset);
int ffk_dropout_backward(ffk_stream_t stream, int dtype,
                         void const *output_grad, void *input_grad,
                         int64_t num_elements, float rate, uint64_t seed,
                         uint64_t offset, int accumulate);
/* The keep mask itself (1 byte per element), for bit-exact checks. */
int ffk_dropout_mask(ffk_stream_t stream, uint8_t *mask, int64_t num_elements,
                     float rate, uint64_t seed, uint64_t offset);
/* Dropout fused with a neighbouring operator.  No counterpart in the
 * reference, whose executor launches one kernel per operator
 * (lib/local-execution/src/local-execution/computation_graph_instance.cc);
 * for executors that find the pair in their graph (the step driver of this
 * library's host mirror does).  Each entry produces exactly the bits of the
 * two separate entries run one after the other (the intermediate is rounded
 * to the storage type where the first operator would have stored it) without
 * the intermediate's trip through memory.  FLOAT or BF16; pointers 16-byte
 * aligned, num_elements a multiple of 8 (BF16) or 4 (FLOAT), offset a
 * multiple of 8 -- anything else is FFK_ERR_INVALID_ARGUMENT and the caller
 * runs the separate operators.
 *   ffk_dropout_add_forward:  output = residual + dropout(input)
 *   ffk_gelu_dropout_forward: output = dropout(GELU(input))
 *   ffk_dropout_gelu_backward: input_grad = dropout_backward(output_grad)
 *                                           * GELU'(gelu_input)             */
int ffk_dropout_add_forward(ffk_stream_t stream, int dtype, void const *input,
                            void const *residual, void *output,
                            int64_t num_elements, float rate, uint64_t seed,
                            uint64_t offset);
int ffk_gelu_dropout_forward(ffk_stream_t stream, int dtype, void const *input,
                             void *output, int64_t num_elements, float rate,
                             uint64_t seed, uint64_t offset);
int ffk_dropout_gelu_backward(ffk_stream_t stream, int dtype,
                              void const *output_grad, void const *gelu_input,
                              void *input_grad, int64_t num_elements,
                              float rate, uint64_t seed, uint64_t offset);

/* Linear with the GELU and the dropout that follow it, and the matching
 * backward.  No counterpart in the reference (one kernel per operator, as
 * above): the sequence is Linear forward (linear_kernels.cu:110-178) ->
 * ElementUnary GELU -> Dropout, and on the way back Dropout backward -> GELU
 * backward behind the input-gradient GEMM of the next Linear's backward
 * (linear_kernels.cu:214-303).  The element-wise operators are applied to the
 * GEMM's output tile while it is stored, so their intermediates never make a
 * trip through memory; results are the bits of the separate entries run one
 * after the other.  BF16 only, shapes that run on the pipelined GEMM tiles
 * (batch and the GEMM's output width multiples of 128 with at least 128 tiles,
 * reduction length a multiple of 64, 16-byte aligned tensors, offset a
 * multiple of 8); anything else is FFK_ERR_UNSUPPORTED before any kernel is
 * launched, and the caller runs the separate operators.
 *   ffk_linear_gelu_dropout_forward:
 *     output [batch, out_dim] = input . weight^T + bias   (kept for backward)
 *     dropped [batch, out_dim] = dropout(GELU(output))
 *   ffk_linear_dropout_add_forward:
 *     output [batch, out_dim] = residual + dropout(input . weight^T + bias);
 *     Linear's own output is not stored (no backward reads it)
 *   ffk_linear_backward_dropout_gelu: Linear backward without activation
 *     (arguments as ffk_linear_backward) of a Linear whose input [batch,
 *     in_dim] was dropout(GELU(gelu_input)):
 *     input_grad = dropout_backward(output_grad . weight) * GELU'(gelu_input);
 *     FFK_ACC_INPUT is not allowed.                                          */
int ffk_linear_gelu_dropout_forward(ffk_stream_t stream, int dtype,
                                    void const *input, void *output,
                                    void *dropped, void const *weight,
                                    void const *bias, int64_t batch,
                                    int64_t in_dim, int64_t out_dim, float rate,
                                    uint64_t seed, uint64_t offset);
int ffk_linear_dropout_add_forward(ffk_stream_t stream, int dtype,
                                   void const *input, void const *residual,
                                   void *output, void const *weight,
                                   void const *bias, int64_t batch,
                                   int64_t in_dim, int64_t out_dim, float rate,
                                   uint64_t seed, uint64_t offset);
int ffk_linear_backward_dropout_gelu(
    ffk_stream_t stream, int dtype, void const *output_grad, void const *input,
    void const *gelu_input, void *input_grad, void const *weight,
    void *weight_grad, void *bias_grad, int64_t batch, int64_t in_dim,
    int64_t out_dim, void *workspace, size_t workspace_bytes, int accumulate,
    float rate, uint64_t seed, uint64_t offset);

/* The bias gradient of a Linear taken where the gradient of its output is
 * produced, instead of by a pass of its own over that gradient.  No
 * counterpart in the reference, whose Linear backward sums the bias gradient
 * with a GEMM against a vector of ones (linear_kernels.cu:294-317).  Results
 * are the bits of the separate entries (the sums are taken over the gradient
 * as stored, in the order ffk_linear_backward takes them).
 *   ffk_dropout_backward_bias_grad: the Dropout that follows a Linear:
 *     input_grad [batch, out_dim] = dropout_backward(output_grad);
 *     bias_grad [out_dim] (+)= its column sums; the Linear's backward is then
 *     called with bias_grad NULL.  FLOAT or BF16.  workspace:
 *     ffk_dropout_backward_bias_grad_workspace_bytes(batch, out_dim).
 *   ffk_linear_backward_dropout_gelu_bias_grad: ffk_linear_backward_dropout_
 *     gelu that also gives the bias gradient of the Linear whose output was
 *     gelu_input: gelu_bias_grad [in_dim] (+)= column sums of input_grad,
 *     taken on the GEMM's tile store.  gelu_bias_workspace:
 *     ffk_dropout_backward_bias_grad_workspace_bytes(batch, in_dim) bytes
 *     that nothing else uses until the call returns (inside
 *     ffk_column_reductions_begin/_end: until _end).
 * FFK_ERR_UNSUPPORTED before any kernel is launched when the shape has no
 * such kernel; the caller then runs the plain entries.                      */
size_t ffk_dropout_backward_bias_grad_workspace_bytes(int64_t batch,
                                                      int64_t out_dim);
int ffk_dropout_backward_bias_grad(ffk_stream_t stream, int dtype,
                                   void const *output_grad, void *input_grad,
                                   int64_t batch, int64_t out_dim,
                                   void *bias_grad, int accumulate_bias,
                                   void *workspace, size_t workspace_bytes,
                                   float rate, uint64_t seed, uint64_t offset);
int ffk_linear_backward_dropout_gelu_bias_grad(
    ffk_stream_t stream, int dtype, void const *output_grad, void const *input,
    void const *gelu_input, void *input_grad, void const *weight,
    void *weight_grad, void *bias_grad, int64_t batch, int64_t in_dim,
    int64_t out_dim, void *workspace, size_t workspace_bytes, int accumulate,
    float rate, uint64_t seed, uint64_t offset, void *gelu_bias_grad,
    int accumulate_gelu_bias, void *gelu_bias_workspace,
    size_t gelu_bias_workspace_bytes);

/* LayerNorm next to the residual add and the dropout of a transformer block.
 * No counterpart in the reference (one kernel per operator, as above): the
 * sequences are Dropout -> ElementBinary add -> LayerNorm going forward
 * (dropout_kernels.cu:67-97, element_binary_kernels.cu:146-248,
 * layer_norm_kernels.cu:412-439) and, going back, the add's backward handing
 * its output gradient to the residual branch, LayerNorm backward adding into
 * it, and the Dropout's backward reading the sum.  Results are the bits of
 * the separate entries run one after the other.  FLOAT or BF16 (the dropout
 * forms BF16 only), rows of a multiple of 8 elements that fit the one-pass
 * kernel, 16-byte aligned tensors, offset a multiple of 8; anything else is
 * FFK_ERR_UNSUPPORTED before any kernel is launched and the caller runs the
 * separate operators.
 *   ffk_dropout_add_layer_norm_forward:
 *     sum [M,N] = residual + dropout(input); output = LayerNorm(sum);
 *     mean / rstd as ffk_layer_norm_forward writes them
 *   ffk_layer_norm_backward_residual: ffk_layer_norm_backward whose input
 *     gradient starts from another tensor:
 *     input_grad = residual + (gradient of the LayerNorm's input), rounded
 *     once -- what FFK_LN_ACC_INPUT gives when input_grad holds a copy of
 *     residual (the gradient of the add's output); gamma_grad / beta_grad as
 *     ffk_layer_norm_backward (accumulate_params != 0 adds into them);
 *     dropped_grad (optional, BF16) = dropout_backward(input_grad as stored),
 *     the gradient of the input of the Dropout whose output was the other
 *     operand of the add that produced the LayerNorm's input.               */
int ffk_dropout_add_layer_norm_forward(ffk_stream_t stream, int dtype,
                                       void const *input, void const *residual,
                                       void *sum, void *output,
                                       void const *gamma, void const *beta,
                                       float *mean, float *rstd, int64_t M,
                                       int64_t N, float eps, float rate,
                                       uint64_t seed, uint64_t offset);
int ffk_layer_norm_backward_residual(
    ffk_stream_t stream, int dtype, void const *output_grad, void const *input,
    float const *mean, float const *rstd, void const *gamma,
    void const *residual, void *input_grad, void *gamma_grad, void *beta_grad,
    int64_t M, int64_t N, void *workspace, size_t workspace_bytes,
    int accumulate_params, void *dropped_grad, float rate, uint64_t seed,
    uint64_t offset);

/* ------------------------------------------------------------------------ */
/* Embedding -- Kernels::Embedding::gpu_forward_kernel / gpu_backward_kernel
 * (embedding_kernels_gpu.h:10-28; lib/kernels/src/cuda/embedding_kernels.cu:
 * 48-317,811-853).  indices [num_bags, bag] (bag == 1 with FFK_AGGR_NONE),
 * index_dtype FFK_INT32 or FFK_INT64; weight [num_entries, dim]; output
 * [num_bags, dim]; weight / output FFK_FLOAT or FFK_BF16 in any pairing, or both
 * FFK_HALF or both FFK_DOUBLE (see ffk_embedding_backward_typed).
 * AVG divides the bag sum by `bag` (not the reference's
 * scale-inside-the-loop, embedding_kernels.cu:85-98).
 * forward:  output[b,:] = sum_j weight[indices[b,j],:]
 * backward: weight_grad[indices[b,j],:] += output_grad[b,:] (* 1/bag for AVG),
 *   fp32 accumulators; weight_grad is always accumulated into.
 *   Without workspace: hardware fp32 atomics, one wave instruction per 64
 *   consecutive floats of a row (order, hence rounding, varies run to run).
 *   With workspace of ffk_embedding_backward_workspace_bytes(num_bags*bag,
 *   num_entries) bytes (256-byte aligned) and dim % 4 == 0: lookups are sorted
 *   by row first and runs of equal rows are summed in registers; only runs
 *   that straddle two walkers' chunks still use atomics.
 *   deterministic == 1 (needs the workspace): every row is summed by one
 *   walker in ascending lookup order, no atomics, bit-reproducible.          */
/* ------------------------------------------------------------------------ */
int ffk_embedding_forward(ffk_stream_t stream, int index_dtype,
                          int weight_dtype, int output_dtype,
                          void const *indices, void *output,
                          void const *weight, int aggr, int64_t num_bags,
                          int64_t bag, int64_t dim, int64_t num_entries);
size_t ffk_embedding_backward_workspace_bytes(int64_t num_indices,
                                              int64_t num_entries);
int ffk_embedding_backward(ffk_stream_t stream, int index_dtype,
                           int output_grad_dtype, void const *indices,
                           void const *output_grad, float *weight_grad,
                           int aggr, int64_t num_bags, int64_t bag, int64_t dim,
                           int64_t num_entries, int deterministic,
                           void *workspace, size_t workspace_bytes);
/* The reference's HALF and DOUBLE instantiations (embedding_kernels.cu:374-449,
 * 491-566 forward; 609-808 backward): table, output and both gradients have one
 * type and all arithmetic is that type's, as there -- ffk_embedding_forward with
 * weight_dtype == output_dtype == FFK_HALF or FFK_DOUBLE sums a bag in that type
 * entry by entry; this entry point adds output_grad (* T(1/bag) for AVG) into
 * weight_grad of the same dtype with atomics (compare-and-swap for HALF).
 * dtype FFK_FLOAT forwards to ffk_embedding_backward without workspace.
 * One thread per element: correct, not tuned (no configuration uses them). */
int ffk_embedding_backward_typed(ffk_stream_t stream, int index_dtype, int dtype,
                                 void const *indices, void const *output_grad,
                                 void *weight_grad, int aggr, int64_t num_bags,
                                 int64_t bag, int64_t dim, int64_t num_entries);

/* ------------------------------------------------------------------------ */
/* Fused (flash-style) scaled-dot-product attention core: the QK^T / softmax /
 * PV contraction that cudnnMultiHeadAttnForward/BackwardData perform inside
 * lib/kernels/src/cuda/ops/attention_kernels.cu:224,261, without the S x S
 * score matrix ever reaching HBM.  dtype FFK_BF16 (head sizes multiples of 8
 * up to 256, strides multiples of 8; 64 and 128 with v_head_dim = head_dim run
 * the tuned kernels) or FFK_FLOAT (the reference's data type; head sizes
 * multiples of 4 up to 256, strides multiples of 4).  q and k have head_dim
 * columns per head, v and o have v_head_dim (qProjSize / vProjSize of
 * lib/kernels/src/cuda/ops/attention_kernels.cu:78-80; the reference's model
 * builders use 256 for both, lib/models/src/models/transformer/transformer.cc:37-38).
 *   q,k,v,o: element (b, s, h, d) at  b*batch_stride + s*seq_stride +
 *   h*(head_dim or v_head_dim) + d  (strides in elements), so the same kernel
 *   reads the [batch, seq, heads*head_dim] projections and a fused QKV buffer.
 *   lse [batch, heads, seq_q] fp32: log-sum-exp of the scaled scores, written
 *   by forward and read by backward.  scale multiplies QK^T (the reference
 *   uses 1.0, attention_kernels.cu:76); causal != 0 masks key index > query
 *   index (aligned top-left when seq_q != seq_kv).
 * backward needs delta [batch, heads, seq_q] fp32 scratch (written inside).  */
/* ------------------------------------------------------------------------ */
typedef struct {
  int64_t batch, heads, seq_q, seq_kv, head_dim;
  int64_t q_batch_stride, q_seq_stride;
  int64_t k_batch_stride, k_seq_stride;
  int64_t v_batch_stride, v_seq_stride;
  int64_t o_batch_stride, o_seq_stride;
  float scale;
  int causal;
  int64_t v_head_dim; /* head size of v, o (and their gradients); 0 = head_dim */
} ffk_attention_desc_t;

int ffk_attention_forward(ffk_stream_t stream, int dtype,
                          ffk_attention_desc_t const *desc, void const *q,
                          void const *k, void const *v, void *o, float *lse);
int ffk_attention_backward(ffk_stream_t stream, int dtype,
                           ffk_attention_desc_t const *desc, void const *q,
                           void const *k, void const *v, void const *o,
                           void const *d_o, float const *lse, float *delta,
                           void *dq, void *dk, void *dv);

/* ------------------------------------------------------------------------ */
/* MultiHeadAttention -- Kernels::MultiHeadAttention::gpu_forward_kernel /
 * gpu_backward_kernel (attention_kernels_gpu.h:27-45; CUDA body
 * lib/kernels/src/cuda/ops/attention_kernels.cu:215-303).
 *   query [B,Sq,qSize], key [B,Skv,kSize], value [B,Skv,vSize],
 *   output [B,Sq,oProjSize].  No bias, no dropout (attention_kernels.cu:73-92).
 *   dtype FFK_FLOAT (the reference's) or FFK_BF16.  q_proj_size must equal
 *   k_proj_size (the reference asserts it, attention_kernels.cu:61);
 *   v_proj_size is free.  FLOAT: multiples of 4 up to 256; BF16: multiples of
 *   8 up to 256 (the reference's model builders use 256,
 *   lib/models/src/models/transformer/transformer.cc:37-38, bert/bert.cc:64-65).
 *   weight blob (defined by this library; the reference never indexes it):
 *     [ W_Q | W_K | W_V | W_O ], W_Q = [heads*qProj, qSize] row-major with
 *     head-major rows (likewise W_K [heads*kProj, kSize], W_V [heads*vProj,
 *     vSize]), W_O = [oProjSize, heads*vProj] row-major.  Total element count
 *     equals the reference's weight tensor (lib/op-attrs/src/op-attrs/ops/
 *     attention.cc:165-185).
 *   The reserve space (ffk_mha_reserve_bytes) holds the projected Q,K,V, the
 *   pre-projection context and the log-sum-exp between forward and backward
 *   plus backward scratch, like MHAPerDeviceState.reserveSpace.  Its layout
 *   follows from the descriptor alone, so backward needs the descriptor forward
 *   had and nothing else.
 * backward: query_grad/key_grad/value_grad are overwritten unless accumulate
 *   (cudnnMultiHeadAttnBackwardData stores them);
 *   key_grad/value_grad may be NULL when key/value alias query (their
 *   gradients are then folded into query_grad, as the reference's task impl
 *   expects, lib/task-spec/src/task-spec/ops/impl/attention.cc:129-133) --
 *   both or neither: one of them NULL alone is FFK_ERR_INVALID;
 *   weight_grad is accumulated into (CUDNN_WGRAD_MODE_ADD).  `accumulate` is
 *   0 / 1 as just described, optionally or-ed with
 *   FFK_MHA_OVERWRITE_WEIGHT_GRAD to store the weight gradient instead of
 *   adding it (a caller that would otherwise clear it first).                */
/* ------------------------------------------------------------------------ */
typedef struct {
  int64_t num_samples, num_heads;
  int64_t q_size, k_size, v_size;
  int64_t q_proj_size, k_proj_size, v_proj_size, o_proj_size;
  int64_t qo_seq_length, kv_seq_length;
  float scale; /* reference: 1.0 */
  int causal;  /* reference: 0   */
} ffk_mha_desc_t;

enum { FFK_MHA_ACC_INPUT_GRADS = 1, FFK_MHA_OVERWRITE_WEIGHT_GRAD = 2 };
size_t ffk_mha_weight_elements(ffk_mha_desc_t const *desc);
size_t ffk_mha_reserve_bytes(ffk_mha_desc_t const *desc, int dtype);
int ffk_mha_forward(ffk_stream_t stream, int dtype, ffk_mha_desc_t const *desc,
                    void const *query, void const *key, void const *value,
                    void const *weight, void *output, void *reserve,
                    size_t reserve_bytes);
int ffk_mha_backward(ffk_stream_t stream, int dtype, ffk_mha_desc_t const *desc,
                     void const *query, void *query_grad, void const *key,
                     void *key_grad, void const *value, void *value_grad,
                     void const *weight, void *weight_grad,
                     void const *output_grad, void *reserve,
                     size_t reserve_bytes, int accumulate);

/* ------------------------------------------------------------------------ */
/* One transformer encoder layer, forward and backward, sequenced over the
 * operator entry points above in the order lib/local-execution runs them
 * (topological FWD pass, then BWD pass in reverse;
 * lib/local-execution/src/local-execution/computation_graph_instance.cc:104-137)
 * for the op list of create_transformer_encoder_layer
 * (lib/models/src/models/transformer/transformer.cc:19-67).
 *   pre_layer_norm == 0: the reference's order
 *       y = LN2(x1 + FFN(x1)),  x1 = LN1(x + MHA(x,x,x))
 *   pre_layer_norm == 1:
 *       x1 = x + drop(MHA(LN1(x)));  y = x1 + drop(W2 drop(act(W1 LN2(x1) + b1)) + b2)
 *   FFN = dense(d_ff, activation, bias) -> dropout -> dense(d_model, bias) -> dropout;
 *   activation: FFK_ACT_RELU (reference) or FFK_ACT_GELU (exact erf GELU as an
 *   ElementUnary op).  MHA: heads x (d_model/heads), no bias, `attn_scale`,
 *   `causal`.  Dropout op i uses seed + i.
 * Tensors: x, y, dy, dx [batch*seq, d_model]; weights as named.  Weight
 * gradients are accumulated into (zero them for a fresh step) unless
 * overwrite_weight_grads is set, in which case every one of them is stored
 * and nothing needs clearing; dx is overwritten.  The workspace keeps every saved activation between the two
 * calls.                                                                     */
/* ------------------------------------------------------------------------ */
typedef struct {
  int64_t batch, seq, d_model, heads, d_ff;
  float dropout_rate;
  uint64_t seed;
  float ln_eps;
  float attn_scale;
  int causal;
  int pre_layer_norm;
  int activation;
  int overwrite_weight_grads; /* 0: add into the weight gradients (reference GPU semantics) */
} ffk_encoder_layer_desc_t;

typedef struct {
  void *ln1_gamma, *ln1_beta; /* [d_model] */
  void *attn_weight;          /* ffk_mha_weight_elements() */
  void *ln2_gamma, *ln2_beta; /* [d_model] */
  void *w1, *b1;              /* [d_ff, d_model], [d_ff] */
  void *w2, *b2;              /* [d_model, d_ff], [d_model] */
} ffk_encoder_layer_params_t;

size_t ffk_encoder_layer_workspace_bytes(ffk_encoder_layer_desc_t const *desc,
                                         int dtype);
int ffk_encoder_layer_forward(ffk_stream_t stream, int dtype,
                              ffk_encoder_layer_desc_t const *desc,
                              ffk_encoder_layer_params_t const *weights,
                              void const *x, void *y, void *workspace,
                              size_t workspace_bytes);
int ffk_encoder_layer_backward(ffk_stream_t stream, int dtype,
                               ffk_encoder_layer_desc_t const *desc,
                               ffk_encoder_layer_params_t const *weights,
                               ffk_encoder_layer_params_t const *weight_grads,
                               void const *x, void const *dy, void *dx,
                               void *workspace, size_t workspace_bytes);

/* Between _begin and _end, on the calling thread, the last step of every bias
 * gradient (ffk_linear_backward) and LayerNorm parameter gradient
 * (ffk_layer_norm_backward) -- a column sum over a few hundred partial rows,
 * microseconds of launch latency for almost no work -- is not launched but
 * collected (up to 8; further ones run at once); _end runs the collected ones
 * as ONE launch on `stream`, which must be the stream the operators ran on.
 * Until then their outputs are not written, and each collected call must have
 * been given workspace of its own (the partial sums stay there).  No
 * counterpart in the reference, which launches every kernel separately; for
 * executors that run a whole backward pass (the step driver of the host
 * mirror does this).  ffk_encoder_layer_backward does the same internally.   */
int ffk_column_reductions_begin(void);
int ffk_column_reductions_end(ffk_stream_t stream);

/* ------------------------------------------------------------------------ */
/* Optimizer updates -- sgd_update_task / adam_update_task
 * (lib/kernels/include/kernels/optimizer_kernels.h:11-36; CUDA bodies
 * lib/kernels/src/cuda/optimizer_kernels.cu:23-44,111-133; CPU SGD
 * lib/kernels/src/kernels/optimizer_kernels_cpu.cc:10-60).
 *   SGD : gt = g + wd*W; if momentum > 0 { V = V*momentum + gt;
 *         gt = nesterov ? gt + momentum*V : V }; W -= lr*gt
 *   Adam: gt = g + wd*W; M = b1*M + (1-b1)*gt; V = b2*V + (1-b2)*gt*gt;
 *         W -= alpha_t * M / (sqrt(V) + epsilon)    (alpha_t is the caller's
 *         bias-corrected step, as in the reference)
 * Every step is a separately rounded fp32 operation, matching the reference's
 * CPU evaluation.  weight, sgd_v, adam_v, adam_m: fp32 [num_elements].
 * weight_grad: grad_dtype FFK_FLOAT or FFK_BF16, [num_replicas][num_elements];
 * replicas are summed in order (the parameter-server launcher's first step;
 * unlike it, the sum is not written back into replica 0).  sgd_v must be given
 * exactly when momentum > 0.  weight_lowp: optional bf16 copy of the updated
 * weights written in the same pass (NULL: none); no reference counterpart.    */
int ffk_sgd_update(ffk_stream_t stream, int grad_dtype, float lr, float momentum,
                   int nesterov, float weight_decay, void const *weight_grad,
                   int64_t num_elements, int num_replicas, float *weight,
                   float *sgd_v, void *weight_lowp);
int ffk_adam_update(ffk_stream_t stream, int grad_dtype, float alpha_t,
                    float beta1, float beta2, float weight_decay, float epsilon,
                    void const *weight_grad, int64_t num_elements,
                    int num_replicas, float *weight, float *adam_v,
                    float *adam_m, void *weight_lowp);

/* ------------------------------------------------------------------------ */
/* Loss-function backward -- *_loss_backward_kernel
 * (lib/kernels/include/kernels/loss_function_kernels.h:9-45; CUDA bodies
 * lib/kernels/src/cuda/loss_function_kernels.cu:21-139).  fp32; the volumes
 * are element counts and must be equal.
 *   sparse categorical CE: logit_grad[s,c] = (logit[s,c] - [c == label[s/k]])
 *                          * (scale_factor * k) for the first num_samples rows
 *                          of num_classes, plain logit * scale beyond them;
 *                          labels outside [0, num_classes) subtract nothing
 *                          (the reference writes out of bounds for them)
 *   categorical CE, MSE  : logit_grad = (logit - label) * scale_factor
 *   identity             : loss_grad = 1 * scale_factor                      */
int ffk_sparse_categorical_crossentropy_loss_backward(
    ffk_stream_t stream, float *logit_grad, float const *logit, int const *label,
    int64_t logit_volume, int64_t logit_grad_volume, int num_samples,
    int num_classes, int k, float scale_factor);
int ffk_categorical_crossentropy_loss_backward(
    ffk_stream_t stream, float *logit_grad, float const *logit, float const *label,
    int64_t logit_volume, int64_t logit_grad_volume, float scale_factor);
int ffk_mean_squared_error_avg_loss_backward(
    ffk_stream_t stream, float *logit_grad, float const *logit, float const *label,
    int64_t logit_volume, int64_t logit_grad_volume, float scale_factor);
int ffk_identity_loss_backward(ffk_stream_t stream, float *loss_grad,
                               float const *loss, int64_t loss_volume,
                               int64_t loss_grad_volume, float scale_factor);

/* ------------------------------------------------------------------------ */
/* Cast -- Kernels::Cast::gpu_forward_kernel / gpu_backward_kernel
 * (cast_kernels_gpu.h; lib/kernels/src/cuda/ops/cast_kernels.cu:25-37).
 *   forward : output[i] = (ODT) input[i]
 *   backward: input_grad[i] = (ODT) output_grad[i] + input_grad[i]
 * Any pair of FFK_BOOL, FFK_INT32, FFK_INT64, FFK_HALF, FFK_FLOAT, FFK_DOUBLE,
 * FFK_BF16; static_cast semantics, float -> bf16/half rounds to nearest even. */
int ffk_cast_forward(ffk_stream_t stream, int input_dtype, int output_dtype,
                     void const *input, void *output, int64_t num_elements);
int ffk_cast_backward(ffk_stream_t stream, int output_grad_dtype,
                      int input_grad_dtype, void const *output_grad,
                      void *input_grad, int64_t num_elements);

/* ------------------------------------------------------------------------ */
/* Concat -- Kernels::Concat::gpu_forward_kernel / gpu_backward_kernel
 * (lib/kernels/include/kernels/concat_kernels.h:9-17; lib/kernels/src/cuda/
 * ops/concat_kernels.cu:22-97).  With the concatenation axis at position a,
 * num_blocks = product of the dims before a and input_blk_elems[i] = product
 * of input i's dims from a on; the output row is the inputs' rows one after
 * another.  All inputs move in one launch (any number of inputs, any data
 * type; pointer arrays are host memory).
 * backward: input_grads[i] (+)= the matching slice of output_grad; the
 *   reference adds (add_with_stride) = accumulate 1 (float and bf16 only),
 *   accumulate 0 overwrites (any data type).                                 */
/* ------------------------------------------------------------------------ */
int ffk_concat_forward(ffk_stream_t stream, int dtype, void *output,
                       void const *const *inputs,
                       int64_t const *input_blk_elems, int num_inputs,
                       int64_t num_blocks);
int ffk_concat_backward(ffk_stream_t stream, int dtype, void const *output_grad,
                        void *const *input_grads,
                        int64_t const *input_blk_elems, int num_inputs,
                        int64_t num_blocks, int accumulate);

/* Split -- Kernels::Split::gpu_forward_kernel / gpu_backward_kernel
 * (lib/kernels/include/kernels/split_kernels.h:9-25; lib/kernels/src/cuda/ops/
 * split_kernels.cu): Concat read the other way.  outputs[i] takes its column
 * window of every input row; backward: input_grad (+)= the output gradients
 * side by side (the reference adds, add_with_stride = accumulate 1).         */
int ffk_split_forward(ffk_stream_t stream, int dtype, void *const *outputs,
                      void const *input, int64_t const *output_blk_elems,
                      int num_outputs, int64_t num_blocks);
int ffk_split_backward(ffk_stream_t stream, int dtype, void *input_grad,
                       void const *const *output_grads,
                       int64_t const *output_blk_elems, int num_outputs,
                       int64_t num_blocks, int accumulate);

/* ------------------------------------------------------------------------ */
/* Transpose -- Kernels::Transpose::gpu_forward_kernel / gpu_backward_kernel
 * (lib/kernels/include/kernels/transpose_kernels.h:11-19; lib/kernels/src/
 * cuda/ops/transpose_kernels.cu:27-110).  Dims in FF order (dim 0 outermost);
 * output dim i is input dim perm[i], up to 8 dims, any data type.
 * backward: input_grad (+)= output_grad moved back through the inverse
 *   permutation; accumulate 1 (the reference's intent, float and bf16) adds,
 *   0 stores.  input_dims / perm describe the FORWARD transpose in both calls. */
/* ------------------------------------------------------------------------ */
int ffk_transpose_forward(ffk_stream_t stream, int dtype, void const *input,
                          void *output, int num_dims, int64_t const *input_dims,
                          int const *perm);
int ffk_transpose_backward(ffk_stream_t stream, int dtype,
                           void const *output_grad, void *input_grad,
                           int num_dims, int64_t const *input_dims,
                           int const *perm, int accumulate);

/* ------------------------------------------------------------------------ */
/* Gather -- Kernels::Gather::gpu_forward_kernel / gpu_backward_kernel
 * (lib/kernels/include/kernels/gather_kernels.h:12-30; lib/kernels/src/cuda/
 * ops/gather_kernels.cu:23-190).  Tensors viewed as [outer, dim_size, stride]
 * around the gathered dim; index has the output's shape, int32 or int64:
 *   output[o, j, s] = input[o, index[o, j, s], s]
 * (an index outside [0, input_dim_size) yields 0 / is skipped).  Forward moves
 * any data type; backward adds float gradients into input_grad: with hardware
 * atomics like the reference, or, along the innermost dim (stride 1) into rows
 * of at most 64 KB, summed per row in LDS first.  The order of the adds is
 * not fixed in either form.                                                  */
/* ------------------------------------------------------------------------ */
int ffk_gather_forward(ffk_stream_t stream, int dtype, int index_dtype,
                       void const *input, void const *index, void *output,
                       int64_t outer, int64_t input_dim_size,
                       int64_t output_dim_size, int64_t stride);
int ffk_gather_backward(ffk_stream_t stream, int index_dtype,
                        float const *output_grad, void const *index,
                        float *input_grad, int64_t outer,
                        int64_t input_dim_size, int64_t output_dim_size,
                        int64_t stride);

#ifdef __cplusplus
}
#endif
#endif /* FFK_H */
