// ElementBinary forward/backward for gfx950 (reference: cudnnOpTensor /
// cudnnAddTensor / cudnnReduceTensor call-throughs and
// elewise_binary_backward_kernel, lib/kernels/src/cuda/ops/
// element_binary_kernels.cu:27-81,150-427).  Single pass, 16 B per lane.
#include "elementwise.h"

namespace ffk {

template <int OP>
struct BinaryFwd {
  __device__ __forceinline__ void operator()(float const (&x)[2],
                                             float (&y)[1]) const {
    float l = x[0], r = x[1];
    float o;
    if (OP == FFK_OP_EW_ADD) o = l + r;
    else if (OP == FFK_OP_EW_SUB) o = l - r;
    else if (OP == FFK_OP_EW_MUL) o = l * r;
    else if (OP == FFK_OP_EW_DIV) o = l / r;
    else if (OP == FFK_OP_EW_MAX) o = fmaxf(l, r);
    else o = fminf(l, r);
    y[0] = o;
  }
};

// in = (out_grad, lhs, rhs[, old lhs_grad, old rhs_grad]); out = (dl, dr).
// Same case analysis as elewise_binary_backward_kernel with alpha = 1 and
// beta = ACC (element_binary_kernels.cu:36-76).
template <int OP, bool ACC, bool NEED_OPERANDS>
struct BinaryBwd {
  static constexpr int kIn = (NEED_OPERANDS ? 3 : 1) + (ACC ? 2 : 0);
  __device__ __forceinline__ void operator()(float const (&in)[kIn],
                                             float (&out)[2]) const {
    float g = in[0];
    float l = NEED_OPERANDS ? in[1] : 0.0f;
    float r = NEED_OPERANDS ? in[2] : 0.0f;
    float dl, dr;
    if (OP == FFK_OP_EW_ADD) { dl = g; dr = g; }
    else if (OP == FFK_OP_EW_SUB) { dl = g; dr = -g; }
    else if (OP == FFK_OP_EW_MUL) { dl = g * r; dr = g * l; }
    else if (OP == FFK_OP_EW_DIV) { dl = g / r; dr = -g * l / (r * r); }
    else if (OP == FFK_OP_EW_MAX) { dl = l >= r ? g : 0.0f; dr = r >= l ? g : 0.0f; }
    else { dl = l <= r ? g : 0.0f; dr = r <= l ? g : 0.0f; }
    if (ACC) {
      dl += in[kIn - 2];
      dr += in[kIn - 1];
    }
    out[0] = dl;
    out[1] = dr;
  }
};

template <typename T, int OP>
static hipError_t binary_fwd(hipStream_t st, void const *l, void const *r,
                             void *o, int64_t n, int64_t nl, int64_t nr) {
  EwArgs<T, 2, 1> a;
  a.in[0] = static_cast<T const *>(l);
  a.in[1] = static_cast<T const *>(r);
  a.in_elems[0] = nl;
  a.in_elems[1] = nr;
  a.out[0] = static_cast<T *>(o);
  a.n = n;
  return ew_launch<T, 2, 1>(st, a, BinaryFwd<OP>{});
}

template <typename T, int OP, bool ACC, bool NEED>
static hipError_t binary_bwd_impl(hipStream_t st, void const *g, void const *l,
                                  void const *r, void *dl, void *dr,
                                  int64_t n) {
  constexpr int kIn = BinaryBwd<OP, ACC, NEED>::kIn;
  EwArgs<T, kIn, 2> a;
  int k = 0;
  a.in[k++] = static_cast<T const *>(g);
  if (NEED) {
    a.in[k++] = static_cast<T const *>(l);
    a.in[k++] = static_cast<T const *>(r);
  }
  if (ACC) {
    a.in[k++] = static_cast<T const *>(dl);
    a.in[k++] = static_cast<T const *>(dr);
  }
  for (int i = 0; i < kIn; i++) a.in_elems[i] = n;
  a.out[0] = static_cast<T *>(dl);
  a.out[1] = static_cast<T *>(dr);
  a.n = n;
  return ew_launch<T, kIn, 2>(st, a, BinaryBwd<OP, ACC, NEED>{});
}

template <typename T, int OP>
static hipError_t binary_bwd(hipStream_t st, void const *g, void const *l,
                             void const *r, void *dl, void *dr, int64_t n,
                             bool acc) {
  constexpr bool need = !(OP == FFK_OP_EW_ADD || OP == FFK_OP_EW_SUB);
  if (acc) return binary_bwd_impl<T, OP, true, need>(st, g, l, r, dl, dr, n);
  return binary_bwd_impl<T, OP, false, need>(st, g, l, r, dl, dr, n);
}

#define FFK_BINARY_OPS(X)                                                      \
  X(FFK_OP_EW_ADD) X(FFK_OP_EW_SUB) X(FFK_OP_EW_MUL) X(FFK_OP_EW_DIV)          \
  X(FFK_OP_EW_MAX) X(FFK_OP_EW_MIN)

}  // namespace ffk

using namespace ffk;

extern "C" int ffk_element_binary_forward(ffk_stream_t stream, int dtype,
                                          int op_type, void const *lhs,
                                          void const *rhs, void *out,
                                          int64_t out_elems, int64_t lhs_elems,
                                          int64_t rhs_elems) {
  FFK_REQUIRE(out_elems >= 0, "element_binary_forward: negative size");
  if (out_elems == 0) return FFK_OK;
  FFK_REQUIRE(lhs && rhs && out, "element_binary_forward: NULL tensor");
  FFK_REQUIRE(lhs_elems > 0 && rhs_elems > 0 && out_elems % lhs_elems == 0 &&
                  out_elems % rhs_elems == 0,
              "element_binary_forward: operand sizes (%lld, %lld) do not "
              "broadcast to %lld",
              (long long)lhs_elems, (long long)rhs_elems, (long long)out_elems);
  hipStream_t st = as_stream(stream);
  hipError_t e = hipErrorInvalidValue;
  bool found = false;
#define X(OPC)                                                                 \
  if (op_type == OPC) {                                                        \
    found = true;                                                              \
    if (dtype == FFK_FLOAT)                                                    \
      e = binary_fwd<float, OPC>(st, lhs, rhs, out, out_elems, lhs_elems,      \
                                 rhs_elems);                                   \
    else if (dtype == FFK_BF16)                                                \
      e = binary_fwd<bf16, OPC>(st, lhs, rhs, out, out_elems, lhs_elems,       \
                                rhs_elems);                                    \
    else                                                                       \
      return fail(FFK_ERR_UNSUPPORTED,                                         \
                  "element_binary_forward: dtype %d not supported", dtype);    \
  }
  FFK_BINARY_OPS(X)
#undef X
  if (!found) {
    return fail(FFK_ERR_UNSUPPORTED,
                "element_binary_forward: unhandled op type %d", op_type);
  }
  FFK_HIP(e);
  return FFK_OK;
}

extern "C" int ffk_element_binary_backward(ffk_stream_t stream, int dtype,
                                           int op_type, void const *out_grad,
                                           void const *lhs, void const *rhs,
                                           void *lhs_grad, void *rhs_grad,
                                           int64_t out_elems, int accumulate) {
  FFK_REQUIRE(out_elems >= 0, "element_binary_backward: negative size");
  if (out_elems == 0) return FFK_OK;
  FFK_REQUIRE(out_grad && lhs_grad && rhs_grad,
              "element_binary_backward: NULL gradient tensor");
  bool need = !(op_type == FFK_OP_EW_ADD || op_type == FFK_OP_EW_SUB);
  FFK_REQUIRE(!need || (lhs && rhs),
              "element_binary_backward: op %d needs lhs and rhs", op_type);
  hipStream_t st = as_stream(stream);
  hipError_t e = hipErrorInvalidValue;
  bool found = false;
#define X(OPC)                                                                 \
  if (op_type == OPC) {                                                        \
    found = true;                                                              \
    if (dtype == FFK_FLOAT)                                                    \
      e = binary_bwd<float, OPC>(st, out_grad, lhs, rhs, lhs_grad, rhs_grad,   \
                                 out_elems, accumulate != 0);                  \
    else if (dtype == FFK_BF16)                                                \
      e = binary_bwd<bf16, OPC>(st, out_grad, lhs, rhs, lhs_grad, rhs_grad,    \
                                out_elems, accumulate != 0);                   \
    else                                                                       \
      return fail(FFK_ERR_UNSUPPORTED,                                         \
                  "element_binary_backward: dtype %d not supported", dtype);   \
  }
  FFK_BINARY_OPS(X)
#undef X
  if (!found) {
    return fail(FFK_ERR_UNSUPPORTED,
                "element_binary_backward: unhandled op type %d", op_type);
  }
  FFK_HIP(e);
  return FFK_OK;
}
