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

// Gradient of ONE operand when an operand is smaller than the output and was broadcast over
// the leading dims (operand index = output index % operand size), for the ops whose broadcast
// case the reference handles (add, sub, mul: cudnnReduceTensor after an optional cudnnOpTensor,
// element_binary_kernels.cu:268-396).  term(i) = the element-wise contribution of output
// element i to this operand's gradient:
//   add: dy   sub: dy (lhs) / -dy (rhs)   mul: dy * other operand
template <typename T, int OP, bool IS_RHS>
__device__ __forceinline__ float broadcast_term(T const *__restrict__ g, T const *__restrict__ other, int64_t i,
                                                int64_t other_elems) {
  float const dy = VecIO<T>::load1(g + i);
  if (OP == FFK_OP_EW_ADD) return dy;
  if (OP == FFK_OP_EW_SUB) return IS_RHS ? -dy : dy;
  return dy * VecIO<T>::load1(other + i % other_elems);
}

// The operand has as many elements as the output: grad[i] (+)= term(i).
template <typename T, int OP, bool IS_RHS>
__global__ __launch_bounds__(256) void binary_bwd_one_full_kernel(T const *__restrict__ g, T const *__restrict__ other,
                                                                  T *grad, int64_t n, int64_t other_elems, int acc) {
  int64_t const stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) {
    float v = broadcast_term<T, OP, IS_RHS>(g, other, i, other_elems);
    if (acc) v += VecIO<T>::load1(grad + i);
    VecIO<T>::store1(grad + i, v);
  }
}

// The operand has E < n elements: grad[j] (+)= sum over the n / E output rows of term(r E + j).
// One workgroup owns 64 columns; its 16 row lanes take rows ry, ry + 16, ... in order and meet
// in LDS in a fixed order, so the sum does not depend on timing.  fp32 accumulation.
template <typename T, int OP, bool IS_RHS>
__global__ __launch_bounds__(1024) void binary_bwd_one_reduce_kernel(T const *__restrict__ g,
                                                                     T const *__restrict__ other, T *grad, int64_t rows,
                                                                     int64_t E, int64_t other_elems, int acc) {
  __shared__ float part[16][64];
  int const cx = threadIdx.x & 63, ry = threadIdx.x >> 6;
  int64_t const col = (int64_t)blockIdx.x * 64 + cx;
  float s = 0.0f;
  if (col < E) {
    for (int64_t r = ry; r < rows; r += 16) s += broadcast_term<T, OP, IS_RHS>(g, other, r * E + col, other_elems);
  }
  part[ry][cx] = s;
  __syncthreads();
  if (ry == 0 && col < E) {
    float t = 0.0f;
#pragma unroll
    for (int k = 0; k < 16; k++) t += part[k][cx];
    if (acc) t += VecIO<T>::load1(grad + col);
    VecIO<T>::store1(grad + col, t);
  }
}

template <typename T, int OP, bool IS_RHS>
static hipError_t binary_bwd_one(hipStream_t st, void const *g, void const *other, void *grad, int64_t n,
                                 int64_t elems, int64_t other_elems, bool acc) {
  T const *gp = static_cast<T const *>(g), *op = static_cast<T const *>(other);
  T *dp = static_cast<T *>(grad);
  if (elems == n) {
    unsigned const blocks = (unsigned)std::min<int64_t>(ceil_div(n, 256), (int64_t)kNumCU * 16);
    binary_bwd_one_full_kernel<T, OP, IS_RHS><<<blocks, 256, 0, st>>>(gp, op, dp, n, other_elems, acc ? 1 : 0);
  } else {
    binary_bwd_one_reduce_kernel<T, OP, IS_RHS><<<(unsigned)ceil_div(elems, 64), 1024, 0, st>>>(
        gp, op, dp, n / elems, elems, other_elems, acc ? 1 : 0);
  }
  return hipGetLastError();
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

extern "C" int ffk_element_binary_backward_broadcast(ffk_stream_t stream, int dtype, int op_type,
                                                     void const *out_grad, void const *lhs, void const *rhs,
                                                     void *lhs_grad, void *rhs_grad, int64_t out_elems,
                                                     int64_t lhs_elems, int64_t rhs_elems, int accumulate) {
  FFK_REQUIRE(out_elems >= 0, "element_binary_backward_broadcast: negative size");
  if (out_elems == 0) return FFK_OK;
  FFK_REQUIRE(out_grad != nullptr, "element_binary_backward_broadcast: NULL output gradient");
  FFK_REQUIRE(lhs_elems > 0 && rhs_elems > 0 && out_elems % lhs_elems == 0 && out_elems % rhs_elems == 0,
              "element_binary_backward_broadcast: operand sizes (%lld, %lld) do not broadcast to %lld",
              (long long)lhs_elems, (long long)rhs_elems, (long long)out_elems);
  if (op_type != FFK_OP_EW_ADD && op_type != FFK_OP_EW_SUB && op_type != FFK_OP_EW_MUL) {
    return fail(FFK_ERR_UNSUPPORTED, "element_binary_backward_broadcast: op %d has no broadcast gradient (add, sub, mul)",
                op_type);
  }
  if (dtype != FFK_FLOAT && dtype != FFK_BF16) {
    return fail(FFK_ERR_UNSUPPORTED, "element_binary_backward_broadcast: dtype %d not supported", dtype);
  }
  FFK_REQUIRE(op_type != FFK_OP_EW_MUL || ((lhs_grad == nullptr || rhs != nullptr) && (rhs_grad == nullptr || lhs != nullptr)),
              "element_binary_backward_broadcast: mul needs the other operand of every gradient asked for");
  hipStream_t st = as_stream(stream);
  bool const acc = accumulate != 0;
#define FFK_ONE(T, OPC)                                                                                        \
  if (lhs_grad != nullptr) FFK_HIP((binary_bwd_one<T, OPC, false>(st, out_grad, rhs, lhs_grad, out_elems, lhs_elems, rhs_elems, acc))); \
  if (rhs_grad != nullptr) FFK_HIP((binary_bwd_one<T, OPC, true>(st, out_grad, lhs, rhs_grad, out_elems, rhs_elems, lhs_elems, acc)));
#define FFK_BY_TYPE(OPC)                      \
  if (dtype == FFK_FLOAT) {                   \
    FFK_ONE(float, OPC)                       \
  } else {                                    \
    FFK_ONE(bf16, OPC)                        \
  }
  if (op_type == FFK_OP_EW_ADD) {
    FFK_BY_TYPE(FFK_OP_EW_ADD)
  } else if (op_type == FFK_OP_EW_SUB) {
    FFK_BY_TYPE(FFK_OP_EW_SUB)
  } else {
    FFK_BY_TYPE(FFK_OP_EW_MUL)
  }
#undef FFK_BY_TYPE
#undef FFK_ONE
  return FFK_OK;
}
