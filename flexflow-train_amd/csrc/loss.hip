// Loss-function backward kernels for gfx950 (reference: lib/kernels/src/cuda/
// loss_function_kernels.cu:21-139).  The reference runs a copy or a difference
// kernel followed by a scale kernel; here each loss is one pass that does the
// same fp32 operations in the same order (subtract, then multiply by the scale),
// so the values are identical.  fp32 only, as in the reference.
#include "ffk_common.h"

namespace ffk {

constexpr int kLossThreads = 256;

// Each lane handles four consecutive elements with 16-byte accesses when the
// tensors are 16-byte aligned (`vec`), one element otherwise.

// logit_grad[s, c] = (logit[s, c] - [c == label[s / k]]) * (scale * k)
// (copy, then `logit_grad[i * num_classes + label[i / k]] -= 1`, then
// scale_kernel(.., 0, scale_factor * k): loss_function_kernels.cu:21-31,59-84)
template <bool VEC>
__global__ __launch_bounds__(kLossThreads) void sparse_cce_backward_kernel(
    float *__restrict__ dlogit, float const *__restrict__ logit,
    int const *__restrict__ label, int64_t num_samples, int64_t num_classes,
    int k, int64_t volume, float scale) {
  constexpr int V = VEC ? 4 : 1;
  int64_t const i = ((int64_t)blockIdx.x * kLossThreads + threadIdx.x) * V;
  if (i >= volume) return;
  int64_t s = i / num_classes;
  int64_t c = i - s * num_classes;
  if (VEC && i + 4 <= volume) {
    f32x4 v = *reinterpret_cast<f32x4 const *>(logit + i);
    // the row's label is looked up once per row the lane touches (-1: no such sample)
    int64_t hot = s < num_samples ? (int64_t)label[s / k] : -1;
#pragma unroll
    for (int e = 0; e < 4; e++) {
      if (hot == c) v[e] = __fsub_rn(v[e], 1.0f);
      v[e] = __fmul_rn(v[e], scale);
      if (++c == num_classes) {
        c = 0;
        s++;
        hot = s < num_samples ? (int64_t)label[s / k] : -1;
      }
    }
    *reinterpret_cast<f32x4 *>(dlogit + i) = v;
  } else {
    for (int64_t j = i; j < i + V && j < volume; j++) {
      float v = logit[j];
      if (s < num_samples && (int64_t)label[s / k] == c) v = __fsub_rn(v, 1.0f);
      dlogit[j] = __fmul_rn(v, scale);
      if (++c == num_classes) {
        c = 0;
        s++;
      }
    }
  }
}

// (logit - label) * scale: categorical cross-entropy and mean-squared-error
// (loss_function_kernels.cu:33-49)
template <bool VEC>
__global__ __launch_bounds__(kLossThreads) void difference_loss_backward_kernel(
    float *__restrict__ dlogit, float const *__restrict__ logit,
    float const *__restrict__ label, int64_t volume, float scale) {
  constexpr int V = VEC ? 4 : 1;
  int64_t const i = ((int64_t)blockIdx.x * kLossThreads + threadIdx.x) * V;
  if (i >= volume) return;
  if (VEC && i + 4 <= volume) {
    f32x4 const a = *reinterpret_cast<f32x4 const *>(logit + i);
    f32x4 const b = *reinterpret_cast<f32x4 const *>(label + i);
    f32x4 o;
#pragma unroll
    for (int e = 0; e < 4; e++) o[e] = __fmul_rn(__fsub_rn(a[e], b[e]), scale);
    *reinterpret_cast<f32x4 *>(dlogit + i) = o;
  } else {
    for (int64_t j = i; j < i + V && j < volume; j++) {
      dlogit[j] = __fmul_rn(__fsub_rn(logit[j], label[j]), scale);
    }
  }
}

static bool aligned16(void const *a, void const *b, void const *c) {
  return ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) | reinterpret_cast<uintptr_t>(c)) & 15) == 0;
}

// 1 * scale (loss_function_kernels.cu:51-57)
__global__ __launch_bounds__(kLossThreads) void identity_loss_backward_kernel(
    float *__restrict__ dloss, int64_t volume, float scale) {
  int64_t const i = (int64_t)blockIdx.x * kLossThreads + threadIdx.x;
  if (i >= volume) return;
  dloss[i] = __fmul_rn(1.0f, scale);
}

static unsigned loss_blocks(int64_t n) { return (unsigned)ceil_div(n > 0 ? n : 1, kLossThreads); }

}  // namespace ffk

using namespace ffk;

extern "C" int ffk_sparse_categorical_crossentropy_loss_backward(
    ffk_stream_t stream, float *logit_grad, float const *logit, int const *label,
    int64_t logit_volume, int64_t logit_grad_volume, int num_samples,
    int num_classes, int k, float scale_factor) {
  FFK_REQUIRE(logit_volume >= 0 && logit_grad_volume == logit_volume && num_samples >= 0 &&
                  num_classes > 0 && k > 0,
              "sparse_categorical_crossentropy_loss_backward: bad sizes");
  FFK_REQUIRE((int64_t)num_samples * num_classes <= logit_volume,
              "sparse_categorical_crossentropy_loss_backward: num_samples * num_classes exceeds the logits");
  if (logit_volume == 0) return FFK_OK;
  FFK_REQUIRE(logit_grad && logit && label, "sparse_categorical_crossentropy_loss_backward: NULL tensor");
  if (aligned16(logit_grad, logit, nullptr)) {
    sparse_cce_backward_kernel<true><<<loss_blocks(ceil_div(logit_volume, 4)), kLossThreads, 0, as_stream(stream)>>>(
        logit_grad, logit, label, num_samples, num_classes, k, logit_volume, scale_factor * (float)k);
  } else {
    sparse_cce_backward_kernel<false><<<loss_blocks(logit_volume), kLossThreads, 0, as_stream(stream)>>>(
        logit_grad, logit, label, num_samples, num_classes, k, logit_volume, scale_factor * (float)k);
  }
  FFK_CHECK_LAUNCH();
  return FFK_OK;
}

static int difference_loss(char const *who, ffk_stream_t stream, float *logit_grad,
                           float const *logit, float const *label, int64_t logit_volume,
                           int64_t logit_grad_volume, float scale_factor) {
  FFK_REQUIRE(logit_volume >= 0 && logit_grad_volume == logit_volume, "%s: bad sizes", who);
  if (logit_volume == 0) return FFK_OK;
  FFK_REQUIRE(logit_grad && logit && label, "%s: NULL tensor", who);
  if (aligned16(logit_grad, logit, label)) {
    difference_loss_backward_kernel<true><<<loss_blocks(ceil_div(logit_volume, 4)), kLossThreads, 0, as_stream(stream)>>>(
        logit_grad, logit, label, logit_volume, scale_factor);
  } else {
    difference_loss_backward_kernel<false><<<loss_blocks(logit_volume), kLossThreads, 0, as_stream(stream)>>>(
        logit_grad, logit, label, logit_volume, scale_factor);
  }
  FFK_CHECK_LAUNCH();
  return FFK_OK;
}

extern "C" int ffk_categorical_crossentropy_loss_backward(
    ffk_stream_t stream, float *logit_grad, float const *logit, float const *label,
    int64_t logit_volume, int64_t logit_grad_volume, float scale_factor) {
  return difference_loss("categorical_crossentropy_loss_backward", stream, logit_grad, logit, label,
                         logit_volume, logit_grad_volume, scale_factor);
}

extern "C" int ffk_mean_squared_error_avg_loss_backward(
    ffk_stream_t stream, float *logit_grad, float const *logit, float const *label,
    int64_t logit_volume, int64_t logit_grad_volume, float scale_factor) {
  return difference_loss("mean_squared_error_avg_loss_backward", stream, logit_grad, logit, label,
                         logit_volume, logit_grad_volume, scale_factor);
}

extern "C" int ffk_identity_loss_backward(ffk_stream_t stream, float *loss_grad,
                                          float const *loss, int64_t loss_volume,
                                          int64_t loss_grad_volume, float scale_factor) {
  (void)loss;
  FFK_REQUIRE(loss_volume >= 0 && loss_grad_volume == loss_volume, "identity_loss_backward: bad sizes");
  if (loss_volume == 0) return FFK_OK;
  FFK_REQUIRE(loss_grad != nullptr, "identity_loss_backward: NULL tensor");
  identity_loss_backward_kernel<<<loss_blocks(loss_volume), kLossThreads, 0, as_stream(stream)>>>(
      loss_grad, loss_volume, scale_factor);
  FFK_CHECK_LAUNCH();
  return FFK_OK;
}
