// The reference's operator entry points (namespace FlexFlow / Kernels::<Op>),
// each unpacking accessors and per-device state into one C-ABI call.  The CPU
// device branch raises: this library executes on the GPU only.
#include "ffk.h"
#include "kernels/attention_kernels.h"
#include "kernels/dropout_kernels.h"
#include "kernels/element_kernels.h"
#include "kernels/embedding_kernels.h"
#include "kernels/cast_kernels.h"
#include "kernels/concat_kernels.h"
#include "kernels/loss_function_kernels.h"
#include "kernels/optimizer_kernels.h"
#include "kernels/shape_kernels.h"
#include "kernels/layer_norm_kernels.h"
#include "kernels/linear_kernels.h"
#include "kernels/softmax_kernels.h"

namespace FlexFlow {

[[noreturn]] static void no_cpu(char const *who) {
  throw std::runtime_error(std::string(who) + ": NOT_IMPLEMENTED for the CPU device type in this library");
}

static int dt(DataType d) { return static_cast<int>(d); }
static int act_code(std::optional<Activation> const &a) { return a.has_value() ? static_cast<int>(*a) : FFK_ACT_NONE; }

static void require_gpu(GenericTensorAccessorR const &a, char const *who) {
  if (a.device_type != DeviceType::GPU) throw std::runtime_error(std::string(who) + ": accessor is not device-resident");
}

// ---- Linear ---------------------------------------------------------------

std::optional<LinearPerDeviceState> linear_init_kernel(
    DeviceType device_type, device_handle_t const &handle, std::optional<Activation> activation,
    std::optional<RegularizerAttrs> regularizer, bool use_bias, DataType input_type,
    DataType weight_type, DataType output_type, int batch_size, int output_num_channels) {
  if (device_type != DeviceType::GPU) return std::nullopt;
  // the reference asserts "Only L2 regularization is supported" in its backward
  // (src/cuda/ops/linear_kernels.cu:286-288); here the state is refused up front
  if (regularizer.has_value() && !std::holds_alternative<L2RegularizerAttrs>(*regularizer)) {
    throw std::runtime_error("linear_init_kernel: Only L2 regularization is supported");
  }
  LinearPerDeviceState s;
  s.handle = handle.require_for_gpu();
  // ReLU sizes the scratch for any activation (same bytes for all of them)
  s.workspace_bytes = ffk_linear_backward_workspace_bytes(
      dt(output_type), activation.has_value() ? FFK_ACT_RELU : FFK_ACT_NONE, use_bias, batch_size, output_num_channels);
  s.workspace = nullptr;
  if (s.workspace_bytes > 0) check_ffk(ffk_malloc(&s.workspace, s.workspace_bytes), "linear_init_kernel");
  s.activation = activation;
  s.regularizer = regularizer;
  s.use_bias = use_bias;
  s.input_type = input_type;
  s.weight_type = weight_type;
  s.output_type = output_type;
  return s;
}

void linear_forward_kernel(device_stream_t const &stream, std::optional<LinearPerDeviceState> const &state,
                           LinearAttrs const &attrs, GenericTensorAccessorR const &input,
                           GenericTensorAccessorW const &output, GenericTensorAccessorR const &projection,
                           std::optional<GenericTensorAccessorR> const &bias) {
  if (!stream.is_gpu()) no_cpu("linear_forward_kernel");
  if (attrs.use_bias != bias.has_value()) throw std::runtime_error("linear_forward_kernel: use_bias does not match bias");
  require_gpu(input, "linear_forward_kernel");
  (void)state;
  int64_t in_dim = dim_at_idx(input.shape.dims, -1);
  int64_t batch = get_num_elements(input.shape.dims) / in_dim;
  int64_t out_dim = dim_at_idx(projection.shape.dims, 0);
  check_ffk(ffk_linear_forward(stream.require_gpu(), dt(input.shape.data_type), act_code(attrs.activation),
                               input.ptr, output.ptr, projection.ptr, bias ? bias->ptr : nullptr, batch,
                               in_dim, out_dim),
            "linear_forward_kernel");
}

void linear_backward_kernel(device_stream_t const &stream, std::optional<LinearPerDeviceState> const &state,
                            LinearAttrs const &attrs, GenericTensorAccessorR const &output,
                            GenericTensorAccessorR const &output_grad, GenericTensorAccessorR const &input,
                            GenericTensorAccessorW const &input_grad, GenericTensorAccessorR const &projection,
                            GenericTensorAccessorW const &projection_grad,
                            std::optional<GenericTensorAccessorW> const &bias_grad) {
  if (!stream.is_gpu()) no_cpu("linear_backward_kernel");
  if (!state.has_value()) throw std::runtime_error("linear_backward_kernel: per-device state required on the GPU");
  int64_t in_dim = dim_at_idx(input.shape.dims, -1);
  int64_t batch = get_num_elements(input.shape.dims) / in_dim;
  int64_t out_dim = dim_at_idx(projection.shape.dims, 0);
  // Reference GPU semantics: all three gradients accumulate (beta = 1).
  check_ffk(ffk_linear_backward(stream.require_gpu(), dt(input.shape.data_type), act_code(attrs.activation), 0,
                                output.ptr, output_grad.ptr, input.ptr, input_grad.ptr, projection.ptr,
                                projection_grad.ptr, bias_grad ? bias_grad->ptr : nullptr, batch, in_dim, out_dim,
                                state->workspace, state->workspace_bytes, FFK_ACC_ALL),
            "linear_backward_kernel");
  // the regulariser's term, once per call behind the weight-gradient product
  // (src/cuda/ops/linear_kernels.cu:269-290)
  if (state->regularizer.has_value()) {
    auto const *l2 = std::get_if<L2RegularizerAttrs>(&*state->regularizer);
    if (l2 == nullptr) throw std::runtime_error("linear_backward_kernel: Only L2 regularization is supported");
    check_ffk(ffk_linear_l2_regularizer_grad(stream.require_gpu(), dt(projection.shape.data_type), projection.ptr,
                                             projection_grad.ptr, get_num_elements(projection.shape.dims), l2->lambda),
              "linear_backward_kernel (L2 regularizer)");
  }
}

void linear_cleanup_kernel(DeviceType device_type, std::optional<LinearPerDeviceState> &state) {
  if (device_type == DeviceType::GPU && state.has_value() && state->workspace != nullptr) {
    check_ffk(ffk_free(state->workspace), "linear_cleanup_kernel");
    state->workspace = nullptr;
  }
}

// ---- MultiHeadAttention -----------------------------------------------------

namespace Kernels::MultiHeadAttention {

static ffk_mha_desc_t make_desc(MHAPerDeviceState const &s) {
  ffk_mha_desc_t d;
  d.num_samples = s.num_samples; d.num_heads = s.num_heads;
  d.q_size = s.qSize; d.k_size = s.kSize; d.v_size = s.vSize;
  d.q_proj_size = s.qProjSize; d.k_proj_size = s.kProjSize; d.v_proj_size = s.vProjSize;
  d.o_proj_size = s.oProjSize;
  d.qo_seq_length = s.qoSeqLength; d.kv_seq_length = s.kvSeqLength;
  d.scale = s.scale; d.causal = s.causal ? 1 : 0;
  return d;
}

std::optional<MHAPerDeviceState> init_kernel(DeviceType device_type, device_handle_t const &handle,
                                             Allocator &allocator, int num_samples, int num_heads, int qSize,
                                             int kSize, int vSize, int qProjSize, int kProjSize, int vProjSize,
                                             int oProjSize, int qoSeqLength, int kvSeqLength, bool add_bias_kv,
                                             DataType data_type, float scale, bool causal) {
  if (device_type != DeviceType::GPU) return std::nullopt;
  if (add_bias_kv) throw std::runtime_error("MultiHeadAttention: add_bias_kv is not supported");
  MHAPerDeviceState s{handle.require_for_gpu(), 0, 0, num_samples, num_heads, qSize, kSize, vSize, qProjSize,
                      kProjSize, vProjSize, oProjSize, qoSeqLength, kvSeqLength, scale, causal, data_type,
                      nullptr, allocator};
  ffk_mha_desc_t d = make_desc(s);
  s.weightSize = ffk_mha_weight_elements(&d) * size_of_datatype(data_type);
  s.reserveSpaceSize = ffk_mha_reserve_bytes(&d, dt(data_type));
  s.reserveSpace = allocator.allocate(s.reserveSpaceSize);
  return s;
}

std::optional<MHAPerDeviceState> init_kernel(DeviceType device_type, device_handle_t const &handle,
                                             Allocator &allocator, int num_samples, int num_heads, int qSize,
                                             int kSize, int vSize, int qProjSize, int kProjSize, int vProjSize,
                                             int oProjSize, int qoSeqLength, int kvSeqLength, bool add_bias_kv) {
  // reference configuration: fp32 tensors, smScalar = 1.0, full window
  // (src/cuda/ops/attention_kernels.cu:73-92,188-193)
  return init_kernel(device_type, handle, allocator, num_samples, num_heads, qSize, kSize, vSize, qProjSize,
                     kProjSize, vProjSize, oProjSize, qoSeqLength, kvSeqLength, add_bias_kv, DataType::FLOAT,
                     1.0f, false);
}

static void run_forward(device_stream_t const &stream, MHAPerDeviceState const &s, void const *q, void const *k,
                        void const *v, void const *w, void *out) {
  ffk_mha_desc_t d = make_desc(s);
  check_ffk(ffk_mha_forward(stream.require_gpu(), dt(s.data_type), &d, q, k, v, w, out, s.reserveSpace,
                            s.reserveSpaceSize),
            "MultiHeadAttention::forward_kernel");
}

void forward_kernel(device_stream_t const &stream, std::optional<MHAPerDeviceState> const &state,
                    float const *q, float const *k, float const *v, float const *w, float *out) {
  if (!stream.is_gpu()) no_cpu("MultiHeadAttention::forward_kernel");
  if (state.value().data_type != DataType::FLOAT) throw std::runtime_error("MultiHeadAttention: float pointers with a state that is not FLOAT");
  run_forward(stream, state.value(), q, k, v, w, out);
}

void forward_kernel(device_stream_t const &stream, std::optional<MHAPerDeviceState> const &state,
                    GenericTensorAccessorR const &q, GenericTensorAccessorR const &k,
                    GenericTensorAccessorR const &v, GenericTensorAccessorR const &w,
                    GenericTensorAccessorW const &out) {
  if (!stream.is_gpu()) no_cpu("MultiHeadAttention::forward_kernel");
  if (q.shape.data_type != state.value().data_type) throw std::runtime_error("MultiHeadAttention: dtype differs from the state's");
  run_forward(stream, *state, q.ptr, k.ptr, v.ptr, w.ptr, out.ptr);
}

static void run_backward(device_stream_t const &stream, MHAPerDeviceState const &s, void const *q, void *dq,
                         void const *k, void *dk, void const *v, void *dv, void const *w, void *dw,
                         void const *dout) {
  ffk_mha_desc_t d = make_desc(s);
  // cudnnMultiHeadAttnBackwardData stores the input gradients, BackwardWeights runs in
  // CUDNN_WGRAD_MODE_ADD (src/cuda/ops/attention_kernels.cu:261-303): the same here
  check_ffk(ffk_mha_backward(stream.require_gpu(), dt(s.data_type), &d, q, dq, k, dk, v, dv, w, dw, dout,
                             s.reserveSpace, s.reserveSpaceSize, 0),
            "MultiHeadAttention::backward_kernel");
}

void backward_kernel(device_stream_t const &stream, std::optional<MHAPerDeviceState> const &state,
                     float const *q, float *dq, float const *k, float *dk, float const *v, float *dv,
                     float const *w, float *dw, float const *dout) {
  if (!stream.is_gpu()) no_cpu("MultiHeadAttention::backward_kernel");
  if (state.value().data_type != DataType::FLOAT) throw std::runtime_error("MultiHeadAttention: float pointers with a state that is not FLOAT");
  run_backward(stream, state.value(), q, dq, k, dk, v, dv, w, dw, dout);
}

void backward_kernel(device_stream_t const &stream, std::optional<MHAPerDeviceState> const &state,
                     GenericTensorAccessorR const &q, GenericTensorAccessorW const &dq,
                     GenericTensorAccessorR const &k, std::optional<GenericTensorAccessorW> const &dk,
                     GenericTensorAccessorR const &v, std::optional<GenericTensorAccessorW> const &dv,
                     GenericTensorAccessorR const &w, GenericTensorAccessorW const &dw,
                     GenericTensorAccessorR const &dout) {
  if (!stream.is_gpu()) no_cpu("MultiHeadAttention::backward_kernel");
  run_backward(stream, state.value(), q.ptr, dq.ptr, k.ptr, dk ? dk->ptr : nullptr, v.ptr,
               dv ? dv->ptr : nullptr, w.ptr, dw.ptr, dout.ptr);
}

void cleanup_kernel(DeviceType device_type, Allocator &allocator, std::optional<MHAPerDeviceState> const &state) {
  if (device_type == DeviceType::GPU && state.has_value() && state->reserveSpace != nullptr) {
    allocator.deallocate(state->reserveSpace);
  }
}

}  // namespace Kernels::MultiHeadAttention

// ---- LayerNorm --------------------------------------------------------------

namespace Kernels::LayerNorm {

std::optional<LayerNormPerDeviceState> init_kernel(DeviceType device_type, device_handle_t const &handle,
                                                   Allocator &allocator, bool elementwise_affine,
                                                   int64_t effective_batch_size, int64_t effective_num_elements,
                                                   float eps) {
  if (device_type != DeviceType::GPU) return std::nullopt;
  LayerNormPerDeviceState s;
  s.handle = handle.require_for_gpu();
  s.elementwise_affine = elementwise_affine;
  s.effective_batch_size = effective_batch_size;
  s.effective_num_elements = effective_num_elements;
  s.eps = eps;
  s.mean = static_cast<float *>(allocator.allocate(sizeof(float) * effective_batch_size));
  s.rstd = static_cast<float *>(allocator.allocate(sizeof(float) * effective_batch_size));
  s.workspace_bytes = ffk_layer_norm_backward_workspace_bytes(effective_batch_size, effective_num_elements);
  s.workspace = allocator.allocate(s.workspace_bytes);
  s.data_type = DataType::FLOAT;
  return s;
}

void forward_kernel(device_stream_t const &stream, std::optional<LayerNormPerDeviceState> const &state,
                    GenericTensorAccessorR const &input, GenericTensorAccessorW const &output,
                    GenericTensorAccessorW const &gamma, GenericTensorAccessorW const &beta) {
  if (!stream.is_gpu()) no_cpu("LayerNorm::forward_kernel");
  LayerNormPerDeviceState const &s = state.value();
  bool affine = s.elementwise_affine;
  check_ffk(ffk_layer_norm_forward(stream.require_gpu(), dt(input.shape.data_type), input.ptr, output.ptr,
                                   affine ? gamma.ptr : nullptr, affine ? beta.ptr : nullptr, s.mean, s.rstd,
                                   s.effective_batch_size, s.effective_num_elements, s.eps),
            "LayerNorm::forward_kernel");
}

void backward_kernel(device_stream_t const &stream, std::optional<LayerNormPerDeviceState> const &state,
                     GenericTensorAccessorR const &output_grad, GenericTensorAccessorR const &input,
                     GenericTensorAccessorW const &input_grad, GenericTensorAccessorR const &gamma,
                     GenericTensorAccessorW const &gamma_grad, GenericTensorAccessorW const &beta_grad) {
  if (!stream.is_gpu()) no_cpu("LayerNorm::backward_kernel");
  LayerNormPerDeviceState const &s = state.value();
  bool affine = s.elementwise_affine;
  check_ffk(ffk_layer_norm_backward(stream.require_gpu(), dt(input.shape.data_type), output_grad.ptr, input.ptr,
                                    s.mean, s.rstd, affine ? gamma.ptr : nullptr, input_grad.ptr,
                                    affine ? gamma_grad.ptr : nullptr, affine ? beta_grad.ptr : nullptr,
                                    s.effective_batch_size, s.effective_num_elements, s.workspace,
                                    s.workspace_bytes, 1),
            "LayerNorm::backward_kernel");
}

void cleanup_kernel(DeviceType, std::optional<LayerNormPerDeviceState> const &) {
  // mean/rstd/workspace belong to the Allocator given to init_kernel
}

}  // namespace Kernels::LayerNorm

// ---- Softmax ----------------------------------------------------------------

namespace Kernels::Softmax {

std::optional<SoftmaxPerDeviceState> init_kernel(DeviceType device_type, device_handle_t const &handle,
                                                 ff_dim_t dim, int n, int c, int h, int w) {
  if (device_type != DeviceType::GPU) return std::nullopt;
  return SoftmaxPerDeviceState{handle.require_for_gpu(), n, c, h, w, dim, DataType::FLOAT};
}

static void run_forward(device_stream_t const &stream, SoftmaxPerDeviceState const &s, int dtype, void const *in,
                        void *out) {
  // cudnnSoftmaxForward(ACCURATE, MODE_CHANNEL) on an (n, c, h, w) view
  check_ffk(ffk_softmax_forward(stream.require_gpu(), dtype, in, out, s.n, s.c, (int64_t)s.h * s.w),
            "Softmax::forward_kernel");
}

void forward_kernel(device_stream_t const &stream, std::optional<SoftmaxPerDeviceState> const &state,
                    float const *in, float *out) {
  if (!stream.is_gpu()) no_cpu("Softmax::forward_kernel");
  run_forward(stream, state.value(), FFK_FLOAT, in, out);
}
void forward_kernel(device_stream_t const &stream, std::optional<SoftmaxPerDeviceState> const &state,
                    GenericTensorAccessorR const &in, GenericTensorAccessorW const &out) {
  if (!stream.is_gpu()) no_cpu("Softmax::forward_kernel");
  run_forward(stream, state.value(), dt(in.shape.data_type), in.ptr, out.ptr);
}
void backward_kernel(device_stream_t const &stream, float const *dout, float *din, size_t n) {
  if (!stream.is_gpu()) no_cpu("Softmax::backward_kernel");
  check_ffk(ffk_softmax_backward_copy(stream.require_gpu(), FFK_FLOAT, dout, din, n), "Softmax::backward_kernel");
}
void backward_kernel(device_stream_t const &stream, std::optional<SoftmaxPerDeviceState> const &state,
                     GenericTensorAccessorR const &output, GenericTensorAccessorR const &output_grad,
                     GenericTensorAccessorW const &input_grad) {
  if (!stream.is_gpu()) no_cpu("Softmax::backward_kernel");
  SoftmaxPerDeviceState const &s = state.value();
  check_ffk(ffk_softmax_backward(stream.require_gpu(), dt(output.shape.data_type), output.ptr, output_grad.ptr,
                                 input_grad.ptr, s.n, s.c, (int64_t)s.h * s.w),
            "Softmax::backward_kernel");
}
void cleanup_kernel(DeviceType, std::optional<SoftmaxPerDeviceState> &) {}

}  // namespace Kernels::Softmax

// ---- Dropout ----------------------------------------------------------------

namespace Kernels::Dropout {

std::optional<DropoutPerDeviceState> init_kernel(DeviceType device_type, device_handle_t const &handle,
                                                 float rate, unsigned long long seed,
                                                 TensorShape const &output_shape, Allocator &) {
  if (device_type != DeviceType::GPU) return std::nullopt;
  return DropoutPerDeviceState{handle.require_for_gpu(), rate, seed, output_shape};
}
void forward_kernel(device_stream_t const &stream, std::optional<DropoutPerDeviceState> const &state,
                    float const *in, float *out) {
  if (!stream.is_gpu()) no_cpu("Dropout::forward_kernel");
  DropoutPerDeviceState const &s = state.value();
  check_ffk(ffk_dropout_forward(stream.require_gpu(), FFK_FLOAT, in, out, get_num_elements(s.output_shape.dims),
                                s.rate, s.seed, 0),
            "Dropout::forward_kernel");
}
void backward_kernel(device_stream_t const &stream, std::optional<DropoutPerDeviceState> const &state,
                     float const *dout, float *din) {
  if (!stream.is_gpu()) no_cpu("Dropout::backward_kernel");
  DropoutPerDeviceState const &s = state.value();
  // cudnnDropoutBackward overwrites dx
  check_ffk(ffk_dropout_backward(stream.require_gpu(), FFK_FLOAT, dout, din,
                                 get_num_elements(s.output_shape.dims), s.rate, s.seed, 0, 0),
            "Dropout::backward_kernel");
}
void forward_kernel(device_stream_t const &stream, std::optional<DropoutPerDeviceState> const &state,
                    GenericTensorAccessorR const &in, GenericTensorAccessorW const &out) {
  if (!stream.is_gpu()) no_cpu("Dropout::forward_kernel");
  DropoutPerDeviceState const &s = state.value();
  check_ffk(ffk_dropout_forward(stream.require_gpu(), dt(in.shape.data_type), in.ptr, out.ptr,
                                get_num_elements(in.shape.dims), s.rate, s.seed, 0),
            "Dropout::forward_kernel");
}
void backward_kernel(device_stream_t const &stream, std::optional<DropoutPerDeviceState> const &state,
                     GenericTensorAccessorR const &dout, GenericTensorAccessorW const &din) {
  if (!stream.is_gpu()) no_cpu("Dropout::backward_kernel");
  DropoutPerDeviceState const &s = state.value();
  check_ffk(ffk_dropout_backward(stream.require_gpu(), dt(dout.shape.data_type), dout.ptr, din.ptr,
                                 get_num_elements(dout.shape.dims), s.rate, s.seed, 0, 0),
            "Dropout::backward_kernel");
}
void cleanup_kernel(DeviceType, Allocator &, std::optional<DropoutPerDeviceState> &) {}

}  // namespace Kernels::Dropout

// ---- ElementUnary / ElementBinary -------------------------------------------

namespace Kernels::ElementUnary {

std::optional<ElementUnaryPerDeviceState> init_kernel(DeviceType device_type, TensorShape const &in,
                                                      TensorShape const &out, ElementUnaryAttrs const &attrs) {
  if (device_type != DeviceType::GPU) return std::nullopt;
  return ElementUnaryPerDeviceState{in, out, attrs.op_type};
}
void forward_kernel(device_stream_t const &stream, std::optional<ElementUnaryPerDeviceState> const &,
                    ElementUnaryAttrs const &attrs, device_handle_t const &, GenericTensorAccessorR const &input,
                    GenericTensorAccessorW const &output) {
  if (!stream.is_gpu()) no_cpu("ElementUnary::forward_kernel");
  check_ffk(ffk_element_unary_forward(stream.require_gpu(), dt(input.shape.data_type),
                                      static_cast<int>(attrs.op_type), attrs.scalar.value_or(0.0f), input.ptr,
                                      output.ptr, get_num_elements(input.shape.dims)),
            "ElementUnary::forward_kernel");
}
void backward_kernel(device_stream_t const &stream, std::optional<ElementUnaryPerDeviceState> const &,
                     ElementUnaryAttrs const &attrs, device_handle_t const &, GenericTensorAccessorR const &output,
                     GenericTensorAccessorR const &output_grad, GenericTensorAccessorR const &input,
                     GenericTensorAccessorW const &input_grad) {
  if (!stream.is_gpu()) no_cpu("ElementUnary::backward_kernel");
  // -1: the reference's per-op `=` / `+=` behaviour
  check_ffk(ffk_element_unary_backward(stream.require_gpu(), dt(input.shape.data_type),
                                       static_cast<int>(attrs.op_type), attrs.scalar.value_or(0.0f), output.ptr,
                                       output_grad.ptr, input.ptr, input_grad.ptr,
                                       get_num_elements(input.shape.dims), -1),
            "ElementUnary::backward_kernel");
}
void cleanup_kernel(DeviceType, std::optional<ElementUnaryPerDeviceState> &) {}

}  // namespace Kernels::ElementUnary

namespace Kernels::ElementBinary {

std::optional<ElementBinaryPerDeviceState> init_kernel(DeviceType device_type, device_handle_t const &handle,
                                                       OperatorType op_type, bool bl, bool br,
                                                       TensorShape const &lhs, TensorShape const &rhs,
                                                       TensorShape const &out) {
  if (device_type != DeviceType::GPU) return std::nullopt;
  // The reference reduces through tensor descriptors built from the shapes, so any
  // size-1 dim of an operand is summed over (src/cuda/ops/element_binary_kernels.cu:85-130,
  // 268-396); the kernels here repeat the smaller operand over the leading dims only.
  if (!broadcasts_over_leading_dims(lhs.dims, out.dims) || !broadcasts_over_leading_dims(rhs.dims, out.dims)) {
    throw std::runtime_error("ElementBinary::init_kernel: broadcast pattern not supported (an operand must equal "
                             "the output's trailing dims after its leading 1s are dropped)");
  }
  return ElementBinaryPerDeviceState{handle.require_for_gpu(), op_type, bl, br, lhs, rhs, out};
}
void forward_kernel(device_stream_t const &stream, std::optional<ElementBinaryPerDeviceState> const &state,
                    float const *lhs, float const *rhs, float *out, OperatorType op_type, bool,
                    device_handle_t const &) {
  if (!stream.is_gpu()) no_cpu("ElementBinary::forward_kernel");
  ElementBinaryPerDeviceState const &s = state.value();
  check_ffk(ffk_element_binary_forward(stream.require_gpu(), FFK_FLOAT, static_cast<int>(op_type), lhs, rhs, out,
                                       get_num_elements(s.output_shape.dims), get_num_elements(s.lhs_shape.dims),
                                       get_num_elements(s.rhs_shape.dims)),
            "ElementBinary::forward_kernel");
}
void backward_kernel(device_stream_t const &stream, std::optional<ElementBinaryPerDeviceState> const &state,
                     float const *dout, float const *lhs, float const *rhs, float *dl, float *dr,
                     OperatorType op_type, bool bl, bool br, device_handle_t const &) {
  if (!stream.is_gpu()) no_cpu("ElementBinary::backward_kernel");
  ElementBinaryPerDeviceState const &s = state.value();
  if (bl || br || dl == nullptr || dr == nullptr) {
    // the reference's broadcast_inputLHS / broadcast_inputRHS branches (a reduction of the output
    // gradient, element_binary_kernels.cu:268-396) and its NULL-gradient checks
    check_ffk(ffk_element_binary_backward_broadcast(stream.require_gpu(), FFK_FLOAT, static_cast<int>(op_type), dout,
                                                    lhs, rhs, dl, dr, get_num_elements(s.output_shape.dims),
                                                    get_num_elements(s.lhs_shape.dims),
                                                    get_num_elements(s.rhs_shape.dims), 1),
              "ElementBinary::backward_kernel");
    return;
  }
  check_ffk(ffk_element_binary_backward(stream.require_gpu(), FFK_FLOAT, static_cast<int>(op_type), dout, lhs, rhs,
                                        dl, dr, get_num_elements(s.output_shape.dims), 1),
            "ElementBinary::backward_kernel");
}
void forward_kernel(device_stream_t const &stream, std::optional<ElementBinaryPerDeviceState> const &state,
                    GenericTensorAccessorR const &lhs, GenericTensorAccessorR const &rhs,
                    GenericTensorAccessorW const &out) {
  if (!stream.is_gpu()) no_cpu("ElementBinary::forward_kernel");
  if (!broadcasts_over_leading_dims(lhs.shape.dims, out.shape.dims) ||
      !broadcasts_over_leading_dims(rhs.shape.dims, out.shape.dims)) {
    throw std::runtime_error("ElementBinary::forward_kernel: broadcast pattern not supported");
  }
  check_ffk(ffk_element_binary_forward(stream.require_gpu(), dt(out.shape.data_type),
                                       static_cast<int>(state.value().op_type), lhs.ptr, rhs.ptr, out.ptr,
                                       get_num_elements(out.shape.dims), get_num_elements(lhs.shape.dims),
                                       get_num_elements(rhs.shape.dims)),
            "ElementBinary::forward_kernel");
}
void backward_kernel(device_stream_t const &stream, std::optional<ElementBinaryPerDeviceState> const &state,
                     GenericTensorAccessorR const &dout, GenericTensorAccessorR const &lhs,
                     GenericTensorAccessorR const &rhs, GenericTensorAccessorW const &dl,
                     GenericTensorAccessorW const &dr) {
  if (!stream.is_gpu()) no_cpu("ElementBinary::backward_kernel");
  check_ffk(ffk_element_binary_backward(stream.require_gpu(), dt(dout.shape.data_type),
                                        static_cast<int>(state.value().op_type), dout.ptr, lhs.ptr, rhs.ptr,
                                        dl.ptr, dr.ptr, get_num_elements(dout.shape.dims), 1),
            "ElementBinary::backward_kernel");
}
void cleanup_kernel(DeviceType, std::optional<ElementBinaryPerDeviceState> const &) {}

}  // namespace Kernels::ElementBinary

// ---- Embedding --------------------------------------------------------------

namespace Kernels::Embedding {

static void bag_geometry(GenericTensorAccessorR const &input, std::optional<AggregateOp> const &aggr,
                         int64_t &num_bags, int64_t &bag) {
  int64_t n = get_num_elements(input.shape.dims);
  bag = aggr.has_value() ? dim_at_idx(input.shape.dims, -1) : 1;
  num_bags = n / bag;
}

void forward_kernel(device_stream_t const &stream, GenericTensorAccessorR const &input,
                    GenericTensorAccessorW const &output, GenericTensorAccessorR const &weight,
                    DataType input_data_type, DataType output_data_type, std::optional<AggregateOp> aggr,
                    num_tensor_dims_t, num_tensor_dims_t, int) {
  if (!stream.is_gpu()) no_cpu("Embedding::forward_kernel");
  if (input.shape.data_type != input_data_type || output.shape.data_type != output_data_type) {
    throw std::runtime_error("Embedding::forward_kernel: data types differ from the accessors'");
  }
  int64_t num_bags, bag;
  bag_geometry(input, aggr, num_bags, bag);
  check_ffk(ffk_embedding_forward(stream.require_gpu(), dt(input_data_type), dt(weight.shape.data_type),
                                  dt(output_data_type), input.ptr, output.ptr, weight.ptr,
                                  aggr.has_value() ? static_cast<int>(*aggr) : FFK_AGGR_NONE, num_bags, bag,
                                  dim_at_idx(weight.shape.dims, 1), dim_at_idx(weight.shape.dims, 0)),
            "Embedding::forward_kernel");
}

void backward_kernel(device_stream_t const &stream, GenericTensorAccessorR const &output,
                     GenericTensorAccessorR const &input, GenericTensorAccessorW const &weight_grad,
                     DataType output_data_type, DataType input_data_type, std::optional<AggregateOp> aggr,
                     num_tensor_dims_t, num_tensor_dims_t, int) {
  if (!stream.is_gpu()) no_cpu("Embedding::backward_kernel");
  int64_t num_bags, bag;
  bag_geometry(input, aggr, num_bags, bag);
  if (weight_grad.shape.data_type == DataType::HALF || weight_grad.shape.data_type == DataType::DOUBLE) {
    // the reference's half / double instantiations: one type throughout (embedding_kernels.cu:609-808)
    if (output_data_type != weight_grad.shape.data_type) {
      throw std::runtime_error("Embedding::backward_kernel: a HALF or DOUBLE weight_grad takes an output gradient of its type");
    }
    check_ffk(ffk_embedding_backward_typed(stream.require_gpu(), dt(input_data_type), dt(output_data_type), input.ptr,
                                           output.ptr, weight_grad.ptr,
                                           aggr.has_value() ? static_cast<int>(*aggr) : FFK_AGGR_NONE, num_bags, bag,
                                           dim_at_idx(weight_grad.shape.dims, 1), dim_at_idx(weight_grad.shape.dims, 0)),
              "Embedding::backward_kernel");
    return;
  }
  if (weight_grad.shape.data_type != DataType::FLOAT) {
    throw std::runtime_error("Embedding::backward_kernel: weight_grad must be FLOAT (fp32 accumulators), HALF or DOUBLE");
  }
  check_ffk(ffk_embedding_backward(stream.require_gpu(), dt(input_data_type), dt(output_data_type), input.ptr,
                                   output.ptr, static_cast<float *>(weight_grad.ptr),
                                   aggr.has_value() ? static_cast<int>(*aggr) : FFK_AGGR_NONE, num_bags, bag,
                                   dim_at_idx(weight_grad.shape.dims, 1), dim_at_idx(weight_grad.shape.dims, 0), 0,
                                   nullptr, 0),
            "Embedding::backward_kernel");
}

}  // namespace Kernels::Embedding
// ---- Optimizer, loss, cast --------------------------------------------------

void sgd_update_task(device_stream_t const &stream, device_handle_t const &, float lr, float momentum,
                     bool nesterov, float weight_decay, GenericTensorAccessorR const &weight_grad,
                     int num_replicas, GenericTensorAccessorW const &weight,
                     std::optional<GenericTensorAccessorW> const &sgd_v) {
  if (sgd_v.has_value() != (momentum > 0.0f)) {
    throw std::runtime_error("sgd_update_task: sgd_v must be given exactly when momentum > 0");
  }
  if (!stream.is_gpu()) no_cpu("sgd_update_task");
  if (weight.shape.data_type != DataType::FLOAT) {
    throw std::runtime_error("sgd_update_task: weights must be FLOAT");
  }
  check_ffk(ffk_sgd_update(stream.require_gpu(), dt(weight_grad.shape.data_type), lr, momentum, nesterov,
                           weight_decay, weight_grad.ptr, get_num_elements(weight.shape.dims), num_replicas,
                           static_cast<float *>(weight.ptr),
                           sgd_v.has_value() ? static_cast<float *>(sgd_v->ptr) : nullptr, nullptr),
            "sgd_update_task");
}

void adam_update_task(device_stream_t const &stream, device_handle_t const &, float alpha_t, float beta1,
                      float beta2, float weight_decay, float epsilon, float const *weight_grad_ptr,
                      size_t size, int num_replicas, float *weight_ptr, float *adam_v_ptr,
                      float *adam_m_ptr) {
  if (!stream.is_gpu()) no_cpu("adam_update_task");
  check_ffk(ffk_adam_update(stream.require_gpu(), FFK_FLOAT, alpha_t, beta1, beta2, weight_decay, epsilon,
                            weight_grad_ptr, (int64_t)size, num_replicas, weight_ptr, adam_v_ptr, adam_m_ptr,
                            nullptr),
            "adam_update_task");
}

void sparse_categorical_crossentropy_loss_backward_kernel(device_stream_t const &stream, float *logit_grad_ptr,
                                                          float const *logit_ptr, int const *label_ptr,
                                                          size_t logit_volume, size_t logit_grad_volume,
                                                          int num_samples, int num_classes, int k,
                                                          float scale_factor) {
  if (!stream.is_gpu()) no_cpu("sparse_categorical_crossentropy_loss_backward_kernel");
  check_ffk(ffk_sparse_categorical_crossentropy_loss_backward(stream.require_gpu(), logit_grad_ptr, logit_ptr,
                                                              label_ptr, (int64_t)logit_volume,
                                                              (int64_t)logit_grad_volume, num_samples,
                                                              num_classes, k, scale_factor),
            "sparse_categorical_crossentropy_loss_backward_kernel");
}

void categorical_crossentropy_loss_backward_kernel(device_stream_t const &stream,
                                                   GenericTensorAccessorW const &logit_grad,
                                                   GenericTensorAccessorR const &logit,
                                                   GenericTensorAccessorR const &label, float scale_factor) {
  if (!stream.is_gpu()) no_cpu("categorical_crossentropy_loss_backward_kernel");
  if (logit.shape.data_type != DataType::FLOAT || label.shape.data_type != DataType::FLOAT ||
      logit_grad.shape.data_type != DataType::FLOAT) {
    throw std::runtime_error("categorical_crossentropy_loss_backward_kernel: tensors must be FLOAT");
  }
  check_ffk(ffk_categorical_crossentropy_loss_backward(
                stream.require_gpu(), static_cast<float *>(logit_grad.ptr),
                static_cast<float const *>(logit.ptr), static_cast<float const *>(label.ptr),
                get_num_elements(logit.shape.dims), get_num_elements(logit_grad.shape.dims), scale_factor),
            "categorical_crossentropy_loss_backward_kernel");
}

void mean_squared_error_avg_loss_backward_kernel(device_stream_t const &stream, float *logit_grad_ptr,
                                                 float const *logit_ptr, float const *label_ptr,
                                                 size_t logit_volume, size_t logit_grad_volume,
                                                 float scale_factor) {
  if (!stream.is_gpu()) no_cpu("mean_squared_error_avg_loss_backward_kernel");
  check_ffk(ffk_mean_squared_error_avg_loss_backward(stream.require_gpu(), logit_grad_ptr, logit_ptr, label_ptr,
                                                     (int64_t)logit_volume, (int64_t)logit_grad_volume,
                                                     scale_factor),
            "mean_squared_error_avg_loss_backward_kernel");
}

void identity_loss_backward_kernel(device_stream_t const &stream, float *loss_grad_ptr, float const *loss_ptr,
                                   size_t loss_volume, size_t loss_grad_volume, float scale_factor) {
  if (!stream.is_gpu()) no_cpu("identity_loss_backward_kernel");
  check_ffk(ffk_identity_loss_backward(stream.require_gpu(), loss_grad_ptr, loss_ptr, (int64_t)loss_volume,
                                       (int64_t)loss_grad_volume, scale_factor),
            "identity_loss_backward_kernel");
}

namespace Kernels::Cast {

void forward_kernel(device_stream_t const &stream, GenericTensorAccessorR const &input,
                    GenericTensorAccessorW const &output) {
  if (!stream.is_gpu()) no_cpu("Cast::forward_kernel");
  check_ffk(ffk_cast_forward(stream.require_gpu(), dt(input.shape.data_type), dt(output.shape.data_type),
                             input.ptr, output.ptr, get_num_elements(input.shape.dims)),
            "Cast::forward_kernel");
}
void backward_kernel(device_stream_t const &stream, GenericTensorAccessorR const &output_grad,
                     GenericTensorAccessorW const &input_grad) {
  if (!stream.is_gpu()) no_cpu("Cast::backward_kernel");
  check_ffk(ffk_cast_backward(stream.require_gpu(), dt(output_grad.shape.data_type),
                              dt(input_grad.shape.data_type), output_grad.ptr, input_grad.ptr,
                              get_num_elements(output_grad.shape.dims)),
            "Cast::backward_kernel");
}

}  // namespace Kernels::Cast

namespace Kernels::Concat {

// [num_blocks, blk] view of a tensor cut at `axis` (concat_kernels.cu:22-31)
static int64_t blk_size(TensorShape const &s, ff_dim_t axis) {
  int64_t n = 1;
  for (int i = axis.value; i < get_num_dims(s.dims); i++) n *= s.dims.ff_ordered[i];
  return n;
}
static int64_t block_count(TensorShape const &s, ff_dim_t axis) {
  int64_t n = 1;
  for (int i = 0; i < axis.value; i++) n *= s.dims.ff_ordered[i];
  return n;
}

template <typename A>
static void check_parts(char const *who, TensorShape const &whole, std::vector<A> const &parts, ff_dim_t axis) {
  if (axis.value < 0 || axis.value >= get_num_dims(whole.dims)) throw std::runtime_error(std::string(who) + ": axis out of range");
  int64_t sum = 0;
  for (A const &p : parts) {
    if (p.shape.data_type != whole.data_type) throw std::runtime_error(std::string(who) + ": data types differ");
    if (get_num_dims(p.shape.dims) != get_num_dims(whole.dims) || block_count(p.shape, axis) != block_count(whole, axis)) {
      throw std::runtime_error(std::string(who) + ": shapes differ outside the axis");
    }
    sum += blk_size(p.shape, axis);
  }
  if (sum != blk_size(whole, axis)) throw std::runtime_error(std::string(who) + ": the parts do not fill the concatenated tensor");
}

void forward_kernel(device_stream_t const &stream, GenericTensorAccessorW const &output,
                    std::vector<GenericTensorAccessorR> const &inputs, ff_dim_t axis) {
  if (!stream.is_gpu()) no_cpu("Concat::forward_kernel");
  check_parts("Concat::forward_kernel", output.shape, inputs, axis);
  std::vector<void const *> ptrs;
  std::vector<int64_t> blks;
  for (GenericTensorAccessorR const &in : inputs) {
    ptrs.push_back(in.ptr);
    blks.push_back(blk_size(in.shape, axis));
  }
  check_ffk(ffk_concat_forward(stream.require_gpu(), dt(output.shape.data_type), output.ptr, ptrs.data(), blks.data(),
                               (int)inputs.size(), block_count(output.shape, axis)),
            "Concat::forward_kernel");
}

void backward_kernel(device_stream_t const &stream, GenericTensorAccessorR const &output_grad,
                     std::vector<GenericTensorAccessorW> const &input_grads, ff_dim_t axis) {
  if (!stream.is_gpu()) no_cpu("Concat::backward_kernel");
  check_parts("Concat::backward_kernel", output_grad.shape, input_grads, axis);
  std::vector<void *> ptrs;
  std::vector<int64_t> blks;
  for (GenericTensorAccessorW const &g : input_grads) {
    ptrs.push_back(g.ptr);
    blks.push_back(blk_size(g.shape, axis));
  }
  check_ffk(ffk_concat_backward(stream.require_gpu(), dt(output_grad.shape.data_type), output_grad.ptr, ptrs.data(),
                                blks.data(), (int)input_grads.size(), block_count(output_grad.shape, axis), 1),
            "Concat::backward_kernel");
}

}  // namespace Kernels::Concat

namespace Kernels::Transpose {

static void check_transpose(char const *who, TransposeAttrs const &attrs, TensorShape const &in, TensorShape const &out) {
  int const nd = get_num_dims(in.dims);
  if ((int)attrs.permutation.size() != nd || get_num_dims(out.dims) != nd || in.data_type != out.data_type) {
    throw std::runtime_error(std::string(who) + ": permutation, input and output disagree");
  }
  for (int i = 0; i < nd; i++) {
    int const p = attrs.permutation[i];
    if (p < 0 || p >= nd || out.dims.ff_ordered[i] != in.dims.ff_ordered[p]) {
      throw std::runtime_error(std::string(who) + ": output dims are not the permuted input dims");
    }
  }
}

void forward_kernel(device_stream_t const &stream, TransposeAttrs const &attrs, GenericTensorAccessorR const &input,
                    GenericTensorAccessorW const &output) {
  if (!stream.is_gpu()) no_cpu("Transpose::forward_kernel");
  check_transpose("Transpose::forward_kernel", attrs, input.shape, output.shape);
  check_ffk(ffk_transpose_forward(stream.require_gpu(), dt(input.shape.data_type), input.ptr, output.ptr,
                                  get_num_dims(input.shape.dims), input.shape.dims.ff_ordered.data(),
                                  attrs.permutation.data()),
            "Transpose::forward_kernel");
}
void backward_kernel(device_stream_t const &stream, TransposeAttrs const &attrs, GenericTensorAccessorR const &out_grad,
                     GenericTensorAccessorW const &in_grad) {
  if (!stream.is_gpu()) no_cpu("Transpose::backward_kernel");
  check_transpose("Transpose::backward_kernel", attrs, in_grad.shape, out_grad.shape);
  check_ffk(ffk_transpose_backward(stream.require_gpu(), dt(in_grad.shape.data_type), out_grad.ptr, in_grad.ptr,
                                   get_num_dims(in_grad.shape.dims), in_grad.shape.dims.ff_ordered.data(),
                                   attrs.permutation.data(), 1),
            "Transpose::backward_kernel");
}

}  // namespace Kernels::Transpose

namespace Kernels::Reshape {

// reshape_kernels.cu: a copy forward, an add backward; the two shapes hold the same elements
void forward_kernel(device_stream_t const &stream, GenericTensorAccessorR const &input,
                    GenericTensorAccessorW const &output) {
  if (!stream.is_gpu()) no_cpu("Reshape::forward_kernel");
  if (get_num_elements(input.shape.dims) != get_num_elements(output.shape.dims) || input.shape.data_type != output.shape.data_type) {
    throw std::runtime_error("Reshape::forward_kernel: shapes hold different element counts or data types");
  }
  check_ffk(ffk_cast_forward(stream.require_gpu(), dt(input.shape.data_type), dt(output.shape.data_type), input.ptr,
                             output.ptr, get_num_elements(input.shape.dims)),
            "Reshape::forward_kernel");
}
void backward_kernel(device_stream_t const &stream, GenericTensorAccessorR const &output,
                     GenericTensorAccessorW const &input) {
  if (!stream.is_gpu()) no_cpu("Reshape::backward_kernel");
  if (get_num_elements(input.shape.dims) != get_num_elements(output.shape.dims) || input.shape.data_type != output.shape.data_type) {
    throw std::runtime_error("Reshape::backward_kernel: shapes hold different element counts or data types");
  }
  check_ffk(ffk_cast_backward(stream.require_gpu(), dt(output.shape.data_type), dt(input.shape.data_type), output.ptr,
                              input.ptr, get_num_elements(input.shape.dims)),
            "Reshape::backward_kernel");
}

}  // namespace Kernels::Reshape

namespace Kernels::Split {

void forward_kernel(device_stream_t const &stream, float **out_ptrs, float const *in_ptr, int const *out_blk_sizes,
                    int in_blk_size, int num_blks, int numOutputs) {
  if (!stream.is_gpu()) no_cpu("Split::forward_kernel");
  std::vector<void *> ptrs(out_ptrs, out_ptrs + numOutputs);
  std::vector<int64_t> blks(out_blk_sizes, out_blk_sizes + numOutputs);
  int64_t sum = 0;
  for (int64_t b : blks) sum += b;
  if (sum != in_blk_size) throw std::runtime_error("Split::forward_kernel: the outputs do not add up to the input block");
  check_ffk(ffk_split_forward(stream.require_gpu(), FFK_FLOAT, ptrs.data(), in_ptr, blks.data(), numOutputs, num_blks),
            "Split::forward_kernel");
}
void backward_kernel(device_stream_t const &stream, float *in_grad_ptr, float const **out_grad_ptr,
                     int const *out_blk_sizes, int in_blk_size, int num_blks, int numOutputs) {
  if (!stream.is_gpu()) no_cpu("Split::backward_kernel");
  std::vector<void const *> ptrs(out_grad_ptr, out_grad_ptr + numOutputs);
  std::vector<int64_t> blks(out_blk_sizes, out_blk_sizes + numOutputs);
  int64_t sum = 0;
  for (int64_t b : blks) sum += b;
  if (sum != in_blk_size) throw std::runtime_error("Split::backward_kernel: the outputs do not add up to the input block");
  check_ffk(ffk_split_backward(stream.require_gpu(), FFK_FLOAT, in_grad_ptr, ptrs.data(), blks.data(), numOutputs,
                               num_blks, 1),
            "Split::backward_kernel");
}

}  // namespace Kernels::Split

namespace Kernels::Gather {

std::optional<GatherPerDeviceState> init_kernel(DeviceType device_type, device_handle_t const &handle, ff_dim_t dim) {
  if (device_type != DeviceType::GPU) return std::nullopt;
  return GatherPerDeviceState{handle.require_for_gpu(), dim};
}

struct GatherView {
  int64_t outer, in_dim, out_dim, stride;
};
static GatherView gather_view(char const *who, ff_dim_t dim, TensorShape const &in, TensorShape const &index) {
  int const nd = get_num_dims(in.dims);
  if (dim.value < 0 || dim.value >= nd || get_num_dims(index.dims) != nd) {
    throw std::runtime_error(std::string(who) + ": dim or ranks out of range");
  }
  GatherView v{1, in.dims.ff_ordered[dim.value], index.dims.ff_ordered[dim.value], 1};
  for (int i = 0; i < nd; i++) {
    if (i != dim.value && in.dims.ff_ordered[i] != index.dims.ff_ordered[i]) {
      throw std::runtime_error(std::string(who) + ": input and index differ outside the gathered dim");
    }
    if (i < dim.value) v.outer *= in.dims.ff_ordered[i];
    if (i > dim.value) v.stride *= in.dims.ff_ordered[i];
  }
  return v;
}

void forward_kernel(device_stream_t const &stream, std::optional<GatherPerDeviceState> const &state,
                    GenericTensorAccessorR const &input, GenericTensorAccessorR const &index,
                    GenericTensorAccessorW const &output) {
  if (!stream.is_gpu()) no_cpu("Gather::forward_kernel");
  if (output.shape.dims != index.shape.dims || output.shape.data_type != input.shape.data_type) {
    throw std::runtime_error("Gather::forward_kernel: the output takes the index's dims and the input's data type");
  }
  GatherView v = gather_view("Gather::forward_kernel", state.value().dim, input.shape, index.shape);
  check_ffk(ffk_gather_forward(stream.require_gpu(), dt(input.shape.data_type), dt(index.shape.data_type), input.ptr,
                               index.ptr, output.ptr, v.outer, v.in_dim, v.out_dim, v.stride),
            "Gather::forward_kernel");
}
void backward_kernel(device_stream_t const &stream, std::optional<GatherPerDeviceState> const &state,
                     GenericTensorAccessorR const &output_grad, GenericTensorAccessorR const &index,
                     GenericTensorAccessorW const &input_grad) {
  if (!stream.is_gpu()) no_cpu("Gather::backward_kernel");
  GatherView v = gather_view("Gather::backward_kernel", state.value().dim, input_grad.shape, index.shape);
  check_ffk(ffk_gather_backward(stream.require_gpu(), dt(index.shape.data_type), output_grad.get_float_ptr(), index.ptr,
                                input_grad.get_float_ptr(), v.outer, v.in_dim, v.out_dim, v.stride),
            "Gather::backward_kernel");
}

}  // namespace Kernels::Gather

}  // namespace FlexFlow
