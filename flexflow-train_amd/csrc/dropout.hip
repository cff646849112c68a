// Dropout forward/backward for gfx950 with a counter-based mask.
//
// The reference delegates to cudnnDropoutForward/Backward, whose generator
// state and reserve space are opaque (lib/kernels/src/cuda/ops/
// dropout_kernels.cu:24-95).  Here the keep mask is a pure function of
// (seed, element index): Philox4x32-10, key = (seed lo, seed hi), counter =
// (block lo, block hi, 0, 0) with block = (offset + i) / 8; element
// e = offset + i uses 16 bits of the block's 128: half (e % 8) % 2 (0 = low)
// of word (e % 8) / 2, and is kept iff half >= ceil(rate * 2^16).  Sixteen
// bits per element keep the generator's integer multiplies (20 per block, all
// quarter-rate) off the critical path: with a 32-bit word per element the
// bf16 passes were bound by them, not by HBM.  Nothing is stored between
// forward and backward: backward regenerates the mask, so both directions
// move 2 tensors only.
#include "ffk_common.h"
#include "fused_ops.h"
#include "dropout_rng.h"
#include <math.h>

namespace ffk {

constexpr int kDropThreads = 256;

// What a fused pass does with the dropped-out value d (rounded to the storage
// type first, as if a separate dropout op had stored it):
//   kDropPlain        y = d
//   kDropAddResidual  y = aux + d            (dropout feeding a residual add)
//   kDropGeluGrad     y = d * GELU'(aux)     (dropout backward feeding the
//                                             backward of a GELU whose input was aux)
//   kDropAfterGelu    y = dropout(GELU(x))   (x is replaced by GELU(x), rounded,
//                                             before the mask is applied)
enum DropMode { kDropPlain = 0, kDropAddResidual = 1, kDropGeluGrad = 2, kDropAfterGelu = 3 };

// offset % 8 == 0, 16-byte aligned pointers: a lane's V elements (8 bf16 or 4
// float) are a whole Philox block or an aligned half of one.
template <typename T, bool ACC, int MODE>
__global__ __launch_bounds__(kDropThreads) void dropout_vec_kernel(
    T const *__restrict__ X, T const *__restrict__ AUX, T *Y, int64_t n, DropoutParams p) {
  constexpr int V = VecIO<T>::kVec;
  int64_t const nvec = n / V;
  int64_t const stride = (int64_t)gridDim.x * kDropThreads;
  for (int64_t i = (int64_t)blockIdx.x * kDropThreads + threadIdx.x; i < nvec; i += stride) {
    float x[V], y[V], aux[V];
    if (MODE == kDropPlain || MODE == kDropAfterGelu) {
      VecIO<T>::load(X + i * V, x);
      if (MODE == kDropAfterGelu) {
#pragma unroll
        for (int e = 0; e < V; e++) x[e] = storage_round<T>(gelu_forward(x[e]));
      }
    } else {
      VecIO<T>::load_stream(X + i * V, x);
      VecIO<T>::load_stream(AUX + i * V, aux);
    }
    if (ACC) VecIO<T>::load(Y + i * V, y);
    static_assert(V == 4 || V == 8, "a lane owns a block of 8 elements or half of one");
    uint64_t const e0 = p.offset + (uint64_t)i * V;
    uint32_t w[4];
    philox4x32_10(e0 >> 3, p.key, w);
    if (V == 4 && (e0 & 4)) {  // upper half of the block
      w[0] = w[2];
      w[1] = w[3];
    }
#pragma unroll
    for (int e = 0; e < V; e++) {
      float v = keep(w, e, p) ? x[e] * p.scale : 0.0f;
      if (MODE == kDropAddResidual) v = storage_round<T>(v) + aux[e];
      if (MODE == kDropGeluGrad) v = storage_round<T>(v) * gelu_derivative(aux[e]);
      y[e] = ACC ? y[e] + v : v;
    }
    VecIO<T>::store(Y + i * V, y);
  }
}

// Any offset / alignment / tail: one element per thread.
template <typename T, bool ACC>
__global__ __launch_bounds__(kDropThreads) void dropout_scalar_kernel(
    T const *__restrict__ X, T *Y, int64_t first, int64_t n, DropoutParams p) {
  int64_t const stride = (int64_t)gridDim.x * kDropThreads;
  for (int64_t i = first + (int64_t)blockIdx.x * kDropThreads + threadIdx.x; i < n; i += stride) {
    uint64_t const e = p.offset + (uint64_t)i;
    uint32_t w[4];
    philox4x32_10(e >> 3, p.key, w);
    float v = keep_dynamic(w, (uint32_t)(e & 7), p) ? VecIO<T>::load1(X + i) * p.scale : 0.0f;
    if (ACC) v += VecIO<T>::load1(Y + i);
    VecIO<T>::store1(Y + i, v);
  }
}

__global__ __launch_bounds__(kDropThreads) void dropout_mask_kernel(
    uint8_t *mask, int64_t n, DropoutParams p) {
  int64_t const stride = (int64_t)gridDim.x * kDropThreads;
  for (int64_t i = (int64_t)blockIdx.x * kDropThreads + threadIdx.x; i < n; i += stride) {
    uint64_t const e = p.offset + (uint64_t)i;
    uint32_t w[4];
    philox4x32_10(e >> 3, p.key, w);
    mask[i] = keep_dynamic(w, (uint32_t)(e & 7), p) ? 1 : 0;
  }
}

// one pass over the tensor (a capped, looping grid measured slower)
static int grid_for(int64_t items) {
  int64_t b = ceil_div(items > 0 ? items : 1, kDropThreads);
  int64_t const cap = (int64_t)1 << 30;
  return (int)(b < cap ? b : cap);
}

template <typename T, bool ACC>
static int dropout_run(hipStream_t st, void const *x, void *y, int64_t n,
                       DropoutParams const &p) {
  constexpr int V = VecIO<T>::kVec;
  T const *X = static_cast<T const *>(x);
  T *Y = static_cast<T *>(y);
  int64_t done = 0;
  if ((p.offset & 7) == 0 && aligned16(x) && aligned16(y) && n >= V) {
    int64_t nvec = n / V;
    dropout_vec_kernel<T, ACC, kDropPlain><<<grid_for(nvec), kDropThreads, 0, st>>>(X, nullptr, Y, n, p);
    FFK_CHECK_LAUNCH();
    done = nvec * V;
  }
  if (done < n) {
    dropout_scalar_kernel<T, ACC><<<grid_for(n - done), kDropThreads, 0, st>>>(X, Y, done, n, p);
    FFK_CHECK_LAUNCH();
  }
  return FFK_OK;
}

// Fused passes used by the encoder-layer sequence; they exist only in the
// vector form and report "not fusable" otherwise so the caller can run the
// separate ops instead.
template <typename T, int MODE>
static int dropout_fused_typed(hipStream_t st, void const *x, void const *aux,
                               void *y, int64_t n, DropoutParams const &p) {
  constexpr int V = VecIO<T>::kVec;
  dropout_vec_kernel<T, false, MODE><<<grid_for(n / V), kDropThreads, 0, st>>>(
      static_cast<T const *>(x), static_cast<T const *>(aux), static_cast<T *>(y), n, p);
  FFK_CHECK_LAUNCH();
  return FFK_OK;
}

bool dropout_fusable(int dtype, void const *x, void const *aux, void const *y,
                     int64_t n, uint64_t offset) {
  int64_t const V = dtype == FFK_BF16 ? 8 : 4;
  return (dtype == FFK_BF16 || dtype == FFK_FLOAT) && n > 0 && n % V == 0 &&
         (offset & 7) == 0 && aligned16(x) && aligned16(aux) && aligned16(y);
}

static int dropout_fused(char const *who, int mode, hipStream_t st, int dtype,
                         void const *x, void const *aux, void *y, int64_t n,
                         float rate, uint64_t seed, uint64_t offset) {
  FFK_REQUIRE(dropout_fusable(dtype, x, aux, y, n, offset), "%s: operands not fusable", who);
  DropoutParams p;
  int rc = make_dropout_params(who, rate, seed, offset, p);
  if (rc != FFK_OK) return rc;
  if (dtype == FFK_FLOAT) {
    if (mode == kDropAfterGelu) return dropout_fused_typed<float, kDropAfterGelu>(st, x, aux, y, n, p);
    return mode == kDropAddResidual ? dropout_fused_typed<float, kDropAddResidual>(st, x, aux, y, n, p)
                                    : dropout_fused_typed<float, kDropGeluGrad>(st, x, aux, y, n, p);
  }
  if (mode == kDropAfterGelu) return dropout_fused_typed<bf16, kDropAfterGelu>(st, x, aux, y, n, p);
  return mode == kDropAddResidual ? dropout_fused_typed<bf16, kDropAddResidual>(st, x, aux, y, n, p)
                                  : dropout_fused_typed<bf16, kDropGeluGrad>(st, x, aux, y, n, p);
}

int gelu_dropout_forward(hipStream_t st, int dtype, void const *x, void *y,
                         int64_t n, float rate, uint64_t seed, uint64_t offset) {
  return dropout_fused("gelu_dropout_forward", kDropAfterGelu, st, dtype, x, nullptr, y, n, rate, seed, offset);
}

int dropout_add_residual(hipStream_t st, int dtype, void const *x,
                         void const *residual, void *y, int64_t n, float rate,
                         uint64_t seed, uint64_t offset) {
  return dropout_fused("dropout_add_residual", kDropAddResidual, st, dtype, x, residual, y, n, rate, seed, offset);
}

int dropout_backward_gelu_backward(hipStream_t st, int dtype, void const *dy,
                                   void const *gelu_input, void *dx, int64_t n,
                                   float rate, uint64_t seed, uint64_t offset) {
  return dropout_fused("dropout_backward_gelu_backward", kDropGeluGrad, st, dtype, dy, gelu_input, dx, n, rate, seed, offset);
}

}  // namespace ffk

using namespace ffk;

extern "C" int ffk_dropout_forward(ffk_stream_t stream, int dtype,
                                   void const *input, void *output,
                                   int64_t num_elements, float rate,
                                   uint64_t seed, uint64_t offset) {
  FFK_REQUIRE(num_elements >= 0, "dropout_forward: negative size");
  DropoutParams p;
  int rc = make_dropout_params("dropout_forward", rate, seed, offset, p);
  if (rc != FFK_OK) return rc;
  if (num_elements == 0) return FFK_OK;
  FFK_REQUIRE(input && output, "dropout_forward: NULL tensor");
  if (dtype == FFK_FLOAT) return dropout_run<float, false>(as_stream(stream), input, output, num_elements, p);
  if (dtype == FFK_BF16) return dropout_run<bf16, false>(as_stream(stream), input, output, num_elements, p);
  return fail(FFK_ERR_UNSUPPORTED, "dropout_forward: dtype %d not supported", dtype);
}

extern "C" int ffk_dropout_backward(ffk_stream_t stream, int dtype,
                                    void const *output_grad, void *input_grad,
                                    int64_t num_elements, float rate,
                                    uint64_t seed, uint64_t offset,
                                    int accumulate) {
  FFK_REQUIRE(num_elements >= 0, "dropout_backward: negative size");
  DropoutParams p;
  int rc = make_dropout_params("dropout_backward", rate, seed, offset, p);
  if (rc != FFK_OK) return rc;
  if (num_elements == 0) return FFK_OK;
  FFK_REQUIRE(output_grad && input_grad, "dropout_backward: NULL tensor");
  hipStream_t st = as_stream(stream);
  if (dtype == FFK_FLOAT) {
    return accumulate ? dropout_run<float, true>(st, output_grad, input_grad, num_elements, p)
                      : dropout_run<float, false>(st, output_grad, input_grad, num_elements, p);
  }
  if (dtype == FFK_BF16) {
    return accumulate ? dropout_run<bf16, true>(st, output_grad, input_grad, num_elements, p)
                      : dropout_run<bf16, false>(st, output_grad, input_grad, num_elements, p);
  }
  return fail(FFK_ERR_UNSUPPORTED, "dropout_backward: dtype %d not supported", dtype);
}

extern "C" int ffk_dropout_add_forward(ffk_stream_t stream, int dtype, void const *input,
                                       void const *residual, void *output, int64_t num_elements,
                                       float rate, uint64_t seed, uint64_t offset) {
  FFK_REQUIRE(input && residual && output, "dropout_add_forward: NULL operand");
  return ffk::dropout_add_residual(as_stream(stream), dtype, input, residual, output, num_elements, rate, seed, offset);
}

extern "C" int ffk_gelu_dropout_forward(ffk_stream_t stream, int dtype, void const *input,
                                        void *output, int64_t num_elements, float rate,
                                        uint64_t seed, uint64_t offset) {
  FFK_REQUIRE(input && output, "gelu_dropout_forward: NULL operand");
  return ffk::gelu_dropout_forward(as_stream(stream), dtype, input, output, num_elements, rate, seed, offset);
}

extern "C" int ffk_dropout_gelu_backward(ffk_stream_t stream, int dtype, void const *output_grad,
                                         void const *gelu_input, void *input_grad,
                                         int64_t num_elements, float rate, uint64_t seed,
                                         uint64_t offset) {
  FFK_REQUIRE(output_grad && gelu_input && input_grad, "dropout_gelu_backward: NULL operand");
  return ffk::dropout_backward_gelu_backward(as_stream(stream), dtype, output_grad, gelu_input, input_grad,
                                             num_elements, rate, seed, offset);
}

extern "C" int ffk_dropout_mask(ffk_stream_t stream, uint8_t *mask,
                                int64_t num_elements, float rate, uint64_t seed,
                                uint64_t offset) {
  FFK_REQUIRE(num_elements >= 0, "dropout_mask: negative size");
  DropoutParams p;
  int rc = make_dropout_params("dropout_mask", rate, seed, offset, p);
  if (rc != FFK_OK) return rc;
  if (num_elements == 0) return FFK_OK;
  FFK_REQUIRE(mask != nullptr, "dropout_mask: NULL mask");
  dropout_mask_kernel<<<grid_for(num_elements), kDropThreads, 0, as_stream(stream)>>>(mask, num_elements, p);
  FFK_CHECK_LAUNCH();
  return FFK_OK;
}
