// ElementUnary forward/backward for gfx950: one coalesced pass, 16 bytes per
// lane per access, the op resolved at compile time (the reference switches on
// the op inside the loop, lib/kernels/src/cuda/ops/element_unary_kernels.cu:
// 104-250, and calls cuDNN for relu/sigmoid/tanh/elu, :255-330).
#include "elementwise.h"

namespace ffk {

#define FFK_SQRT1_2 0.70710678118654752440f
#define FFK_INV_SQRT_2PI 0.39894228040143267794f

template <int OP>
struct UnaryFwd {
  float s;
  __device__ __forceinline__ void operator()(float const (&x)[1],
                                             float (&y)[1]) const {
    float v = x[0];
    float r;
    if (OP == FFK_OP_SCALAR_MULTIPLY) r = v * s;
    else if (OP == FFK_OP_SCALAR_ADD) r = v + s;
    else if (OP == FFK_OP_SCALAR_SUB) r = v - s;
    else if (OP == FFK_OP_SCALAR_TRUE_DIV) r = v / s;
    else if (OP == FFK_OP_POW) r = powf(v, s);
    else if (OP == FFK_OP_EXP) r = expf(v);
    else if (OP == FFK_OP_IDENTITY) r = v;
    else if (OP == FFK_OP_GELU) r = gelu_forward(v);
    else if (OP == FFK_OP_RSQRT) r = 1.0f / sqrtf(v);
    else if (OP == FFK_OP_SIN) r = sinf(v);
    else if (OP == FFK_OP_COS) r = cosf(v);
    else if (OP == FFK_OP_RELU) r = v > 0.0f ? v : 0.0f;
    else if (OP == FFK_OP_SIGMOID) r = 1.0f / (1.0f + expf(-v));
    else if (OP == FFK_OP_TANH) r = tanhf(v);
    else if (OP == FFK_OP_ELU) r = v > 0.0f ? v : s * (expf(v) - 1.0f);
    else r = v;
    y[0] = r;
  }
};

// Which saved tensors an op's gradient reads; the others are never loaded.
template <int OP>
struct UnaryBwdNeeds {
  static constexpr bool kY = OP == FFK_OP_RSQRT || OP == FFK_OP_SIGMOID ||
                             OP == FFK_OP_TANH || OP == FFK_OP_ELU;
  static constexpr bool kX = OP == FFK_OP_POW || OP == FFK_OP_EXP ||
                             OP == FFK_OP_GELU || OP == FFK_OP_GELU_REFERENCE_GRAD ||
                             OP == FFK_OP_SIN || OP == FFK_OP_COS ||
                             OP == FFK_OP_RELU || OP == FFK_OP_ELU;
  static constexpr int kInputs = 1 + (kY ? 1 : 0) + (kX ? 1 : 0);
};

// Backward: inputs are (output_grad[, output][, input][, old input_grad]),
// the optional ones present when UnaryBwdNeeds / ACC say so.
template <int OP, bool ACC>
struct UnaryBwd {
  using Needs = UnaryBwdNeeds<OP>;
  static constexpr int kIn = Needs::kInputs + (ACC ? 1 : 0);
  float s;
  __device__ __forceinline__ void operator()(float const (&in)[kIn],
                                             float (&out)[1]) const {
    float const dy = in[0];
    float const y = Needs::kY ? in[1] : 0.0f;
    float const x = Needs::kX ? in[Needs::kY ? 2 : 1] : 0.0f;
    float g;
    if (OP == FFK_OP_SCALAR_MULTIPLY) g = dy * s;
    else if (OP == FFK_OP_SCALAR_ADD) g = dy;
    else if (OP == FFK_OP_SCALAR_SUB) g = dy;
    else if (OP == FFK_OP_SCALAR_TRUE_DIV) g = dy / s;
    else if (OP == FFK_OP_POW) g = dy * s * powf(x, s - 1.0f);
    else if (OP == FFK_OP_EXP) g = dy * expf(x);
    else if (OP == FFK_OP_IDENTITY) g = dy;
    else if (OP == FFK_OP_GELU)
      // d/dx [x Phi(x)] = Phi(x) + x phi(x)
      g = dy * gelu_derivative(x);
    else if (OP == FFK_OP_GELU_REFERENCE_GRAD)
      // literal text of element_unary_kernels.cu:226-231
      g = dy * (0.5f * erfcf(-x * FFK_SQRT1_2) -
                0.5f * FFK_SQRT1_2 * x * expf(-x * x * 0.5f));
    else if (OP == FFK_OP_RSQRT) g = -0.5f * dy * y * y * y;
    else if (OP == FFK_OP_SIN) g = dy * cosf(x);
    else if (OP == FFK_OP_COS) g = -dy * sinf(x);
    else if (OP == FFK_OP_RELU) g = x > 0.0f ? dy : 0.0f;
    else if (OP == FFK_OP_SIGMOID) g = dy * y * (1.0f - y);
    else if (OP == FFK_OP_TANH) g = dy * (1.0f - y * y);
    else if (OP == FFK_OP_ELU) g = x > 0.0f ? dy : dy * (y + s);
    else g = dy;
    out[0] = ACC ? in[kIn - 1] + g : g;
  }
};

template <typename T, int OP>
static hipError_t unary_fwd(hipStream_t st, float s, void const *in, void *out,
                            int64_t n) {
  EwArgs<T, 1, 1> a;
  a.in[0] = static_cast<T const *>(in);
  a.in_elems[0] = n;
  a.out[0] = static_cast<T *>(out);
  a.n = n;
  return ew_launch<T, 1, 1>(st, a, UnaryFwd<OP>{s});
}

template <typename T, int OP, bool ACC>
static hipError_t unary_bwd_acc(hipStream_t st, float s, void const *y,
                                void const *dy, void const *x, void *dx,
                                int64_t n) {
  using Needs = UnaryBwdNeeds<OP>;
  constexpr int NIN = UnaryBwd<OP, ACC>::kIn;
  EwArgs<T, NIN, 1> a;
  int k = 0;
  a.in[k++] = static_cast<T const *>(dy);
  if (Needs::kY) a.in[k++] = static_cast<T const *>(y);
  if (Needs::kX) a.in[k++] = static_cast<T const *>(x);
  if (ACC) a.in[k++] = static_cast<T const *>(dx);
  for (int i = 0; i < NIN; i++) a.in_elems[i] = n;
  a.out[0] = static_cast<T *>(dx);
  a.n = n;
  return ew_launch<T, NIN, 1>(st, a, UnaryBwd<OP, ACC>{s});
}

template <typename T, int OP>
static hipError_t unary_bwd(hipStream_t st, float s, void const *y,
                            void const *dy, void const *x, void *dx, int64_t n,
                            bool acc) {
  if (acc) return unary_bwd_acc<T, OP, true>(st, s, y, dy, x, dx, n);
  return unary_bwd_acc<T, OP, false>(st, s, y, dy, x, dx, n);
}

// Reference accumulate behaviour per op (element_unary_kernels.cu:172-250:
// `=` for POW, GELU, RSQRT; `+=` otherwise; cuDNN activations use beta = 1).
static bool reference_accumulates(int op) {
  return !(op == FFK_OP_POW || op == FFK_OP_GELU ||
           op == FFK_OP_GELU_REFERENCE_GRAD || op == FFK_OP_RSQRT);
}

#define FFK_UNARY_OPS(X)                                                       \
  X(FFK_OP_SCALAR_MULTIPLY) X(FFK_OP_SCALAR_ADD) X(FFK_OP_SCALAR_SUB)          \
  X(FFK_OP_SCALAR_TRUE_DIV) X(FFK_OP_POW) X(FFK_OP_EXP) X(FFK_OP_IDENTITY)     \
  X(FFK_OP_GELU) X(FFK_OP_RSQRT) X(FFK_OP_SIN) X(FFK_OP_COS) X(FFK_OP_RELU)    \
  X(FFK_OP_SIGMOID) X(FFK_OP_TANH) X(FFK_OP_ELU)

}  // namespace ffk

using namespace ffk;

extern "C" int ffk_element_unary_forward(ffk_stream_t stream, int dtype,
                                         int op_type, float scalar,
                                         void const *input, void *output,
                                         int64_t num_elements) {
  FFK_REQUIRE(num_elements >= 0, "element_unary_forward: negative size");
  if (num_elements == 0) return FFK_OK;
  FFK_REQUIRE(input && output, "element_unary_forward: NULL tensor");
  if (op_type == FFK_OP_GELU_REFERENCE_GRAD) op_type = FFK_OP_GELU;
  hipStream_t st = as_stream(stream);
  hipError_t e = hipErrorInvalidValue;
  bool found = false;
#define X(OPC)                                                                 \
  if (op_type == OPC) {                                                        \
    found = true;                                                              \
    if (dtype == FFK_FLOAT)                                                    \
      e = unary_fwd<float, OPC>(st, scalar, input, output, num_elements);      \
    else if (dtype == FFK_BF16)                                                \
      e = unary_fwd<bf16, OPC>(st, scalar, input, output, num_elements);       \
    else                                                                       \
      return fail(FFK_ERR_UNSUPPORTED,                                         \
                  "element_unary_forward: dtype %d not supported", dtype);     \
  }
  FFK_UNARY_OPS(X)
#undef X
  if (!found) {
    return fail(FFK_ERR_UNSUPPORTED,
                "element_unary_forward: unhandled op type %d", op_type);
  }
  FFK_HIP(e);
  return FFK_OK;
}

extern "C" int ffk_element_unary_backward(ffk_stream_t stream, int dtype,
                                          int op_type, float scalar,
                                          void const *output,
                                          void const *output_grad,
                                          void const *input, void *input_grad,
                                          int64_t num_elements,
                                          int accumulate) {
  FFK_REQUIRE(num_elements >= 0, "element_unary_backward: negative size");
  if (num_elements == 0) return FFK_OK;
  FFK_REQUIRE(output && output_grad && input && input_grad,
              "element_unary_backward: NULL tensor");
  bool acc = accumulate < 0 ? reference_accumulates(op_type) : accumulate != 0;
  hipStream_t st = as_stream(stream);
  hipError_t e = hipErrorInvalidValue;
  bool found = false;
#define X(OPC)                                                                 \
  if (op_type == OPC) {                                                        \
    found = true;                                                              \
    if (dtype == FFK_FLOAT)                                                    \
      e = unary_bwd<float, OPC>(st, scalar, output, output_grad, input,        \
                                input_grad, num_elements, acc);                \
    else if (dtype == FFK_BF16)                                                \
      e = unary_bwd<bf16, OPC>(st, scalar, output, output_grad, input,         \
                               input_grad, num_elements, acc);                 \
    else                                                                       \
      return fail(FFK_ERR_UNSUPPORTED,                                         \
                  "element_unary_backward: dtype %d not supported", dtype);    \
  }
  FFK_UNARY_OPS(X)
  X(FFK_OP_GELU_REFERENCE_GRAD)
#undef X
  if (!found) {
    return fail(FFK_ERR_UNSUPPORTED,
                "element_unary_backward: unhandled op type %d", op_type);
  }
  FFK_HIP(e);
  return FFK_OK;
}
