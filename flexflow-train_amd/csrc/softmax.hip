// Softmax forward / backward for gfx950.
//
// The tensor is viewed as [outer, dim, inner] and normalised over `dim`.
// inner == 1 (softmax over the contiguous last dim) takes the single-pass
// register-resident path: each row is read once, reduced with wave shuffles
// and written once.  inner > 1 (the NCHW "channel" softmax that
// cudnnSoftmaxForward(ACCURATE, MODE_CHANNEL) performs in the reference,
// lib/kernels/src/cuda/ops/softmax_kernels.cu:45-60) takes a strided kernel
// that is coalesced across `inner`.
#include "rowwise.h"

namespace ffk {

template <typename T, int EPT, int WPR, bool STREAM>
__global__ __launch_bounds__(kRowThreads) void softmax_fwd_kernel(
    T const *__restrict__ X, T *__restrict__ Y, int64_t rows, int N) {
  constexpr int V = VecIO<T>::kVec;
  constexpr int RPB = 4 / WPR;
  constexpr int LANES = 64 * WPR;
  __shared__ float smem[2][4][2];
  RowReducer<WPR> red(smem);
  int const nvec = N / V;
  int const lane = WPR == 1 ? (threadIdx.x & 63) : threadIdx.x;
  int64_t const row = (int64_t)blockIdx.x * RPB + (WPR == 1 ? (threadIdx.x >> 6) : 0);
  bool const row_ok = row < rows;
  T const *xr = X + (row_ok ? row : 0) * (int64_t)N;
  float x[EPT][V];
  float mx = -INFINITY;
#pragma unroll
  for (int j = 0; j < EPT; j++) {
    int v = lane + j * LANES;
    if (v < nvec) {
      if (STREAM) {
        VecIO<T>::load_stream(xr + (int64_t)v * V, x[j]);
      } else {
        VecIO<T>::load(xr + (int64_t)v * V, x[j]);
      }
#pragma unroll
      for (int e = 0; e < V; e++) mx = fmaxf(mx, x[j][e]);
    } else {
#pragma unroll
      for (int e = 0; e < V; e++) x[j][e] = -INFINITY;
    }
  }
  mx = red.max(mx);
  float s = 0.0f;
#pragma unroll
  for (int j = 0; j < EPT; j++) {
#pragma unroll
    for (int e = 0; e < V; e++) {
      float p = __expf(x[j][e] - mx);
      x[j][e] = p;
      s += p;
    }
  }
  s = red.sum(s);
  if (!row_ok) return;
  float const inv = 1.0f / s;
  T *yr = Y + row * (int64_t)N;
#pragma unroll
  for (int j = 0; j < EPT; j++) {
    int v = lane + j * LANES;
    if (v < nvec) {
      float y[V];
#pragma unroll
      for (int e = 0; e < V; e++) y[e] = x[j][e] * inv;
      if (STREAM) {
        VecIO<T>::store_stream(yr + (int64_t)v * V, y);
      } else {
        VecIO<T>::store(yr + (int64_t)v * V, y);
      }
    }
  }
}

template <typename T, int EPT, int WPR, bool STREAM>
__global__ __launch_bounds__(kRowThreads) void softmax_bwd_kernel(
    T const *__restrict__ Y, T const *__restrict__ dY, T *__restrict__ dX,
    int64_t rows, int N) {
  constexpr int V = VecIO<T>::kVec;
  constexpr int RPB = 4 / WPR;
  constexpr int LANES = 64 * WPR;
  __shared__ float smem[2][4][2];
  RowReducer<WPR> red(smem);
  int const nvec = N / V;
  int const lane = WPR == 1 ? (threadIdx.x & 63) : threadIdx.x;
  int64_t const row = (int64_t)blockIdx.x * RPB + (WPR == 1 ? (threadIdx.x >> 6) : 0);
  bool const row_ok = row < rows;
  int64_t const r = row_ok ? row : 0;
  float y[EPT][V], dy[EPT][V];
  float dot = 0.0f;
#pragma unroll
  for (int j = 0; j < EPT; j++) {
    int v = lane + j * LANES;
    if (v < nvec) {
      // two input streams read once: cache-bypassing loads
      VecIO<T>::load_stream(Y + r * (int64_t)N + (int64_t)v * V, y[j]);
      VecIO<T>::load_stream(dY + r * (int64_t)N + (int64_t)v * V, dy[j]);
#pragma unroll
      for (int e = 0; e < V; e++) dot += y[j][e] * dy[j][e];
    }
  }
  dot = red.sum(dot);
  if (!row_ok) return;
#pragma unroll
  for (int j = 0; j < EPT; j++) {
    int v = lane + j * LANES;
    if (v < nvec) {
      float o[V];
#pragma unroll
      for (int e = 0; e < V; e++) o[e] = y[j][e] * (dy[j][e] - dot);
      if (STREAM) {
        VecIO<T>::store_stream(dX + row * (int64_t)N + (int64_t)v * V, o);
      } else {
        VecIO<T>::store(dX + row * (int64_t)N + (int64_t)v * V, o);
      }
    }
  }
}

// Strided / generic: one thread per (outer, inner) position walks `dim`.
// Threads of a wave cover consecutive `inner`, so accesses stay coalesced.
// With inner == 1 this is also the fallback for rows that do not fit the
// register-resident kernel.
template <typename T>
__global__ __launch_bounds__(256) void softmax_fwd_strided_kernel(
    T const *__restrict__ X, T *__restrict__ Y, int64_t outer, int64_t dim,
    int64_t inner) {
  int64_t const idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= outer * inner) return;
  int64_t const o = idx / inner, i = idx % inner;
  T const *xp = X + o * dim * inner + i;
  T *yp = Y + o * dim * inner + i;
  float mx = -INFINITY;
  for (int64_t c = 0; c < dim; c++) mx = fmaxf(mx, VecIO<T>::load1(xp + c * inner));
  float s = 0.0f;
  for (int64_t c = 0; c < dim; c++) s += __expf(VecIO<T>::load1(xp + c * inner) - mx);
  float const inv = 1.0f / s;
  for (int64_t c = 0; c < dim; c++) {
    VecIO<T>::store1(yp + c * inner, __expf(VecIO<T>::load1(xp + c * inner) - mx) * inv);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void softmax_bwd_strided_kernel(
    T const *__restrict__ Y, T const *__restrict__ dY, T *__restrict__ dX,
    int64_t outer, int64_t dim, int64_t inner) {
  int64_t const idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= outer * inner) return;
  int64_t const o = idx / inner, i = idx % inner;
  int64_t const base = o * dim * inner + i;
  float dot = 0.0f;
  for (int64_t c = 0; c < dim; c++) {
    dot += VecIO<T>::load1(Y + base + c * inner) * VecIO<T>::load1(dY + base + c * inner);
  }
  for (int64_t c = 0; c < dim; c++) {
    float y = VecIO<T>::load1(Y + base + c * inner);
    VecIO<T>::store1(dX + base + c * inner, y * (VecIO<T>::load1(dY + base + c * inner) - dot));
  }
}

// Long contiguous rows that do not fit in registers: one workgroup per row,
// three passes (the re-reads hit L2 for rows of a few hundred KB).
template <typename T>
__global__ __launch_bounds__(kRowThreads) void softmax_fwd_longrow_kernel(
    T const *__restrict__ X, T *__restrict__ Y, int64_t N) {
  __shared__ float smem[2][4][2];
  RowReducer<4> red(smem);
  T const *xr = X + (int64_t)blockIdx.x * N;
  T *yr = Y + (int64_t)blockIdx.x * N;
  float mx = -INFINITY;
  for (int64_t j = threadIdx.x; j < N; j += kRowThreads) mx = fmaxf(mx, VecIO<T>::load1(xr + j));
  mx = red.max(mx);
  float s = 0.0f;
  for (int64_t j = threadIdx.x; j < N; j += kRowThreads) s += __expf(VecIO<T>::load1(xr + j) - mx);
  float const inv = 1.0f / red.sum(s);
  for (int64_t j = threadIdx.x; j < N; j += kRowThreads) {
    VecIO<T>::store1(yr + j, __expf(VecIO<T>::load1(xr + j) - mx) * inv);
  }
}

template <typename T>
__global__ __launch_bounds__(kRowThreads) void softmax_bwd_longrow_kernel(
    T const *__restrict__ Y, T const *__restrict__ dY, T *__restrict__ dX,
    int64_t N) {
  __shared__ float smem[2][4][2];
  RowReducer<4> red(smem);
  int64_t const base = (int64_t)blockIdx.x * N;
  float dot = 0.0f;
  for (int64_t j = threadIdx.x; j < N; j += kRowThreads) {
    dot += VecIO<T>::load1(Y + base + j) * VecIO<T>::load1(dY + base + j);
  }
  dot = red.sum(dot);
  for (int64_t j = threadIdx.x; j < N; j += kRowThreads) {
    float y = VecIO<T>::load1(Y + base + j);
    VecIO<T>::store1(dX + base + j, y * (VecIO<T>::load1(dY + base + j) - dot));
  }
}

template <typename T>
static int softmax_fwd(hipStream_t st, void const *x, void *y, int64_t outer,
                       int64_t dim, int64_t inner) {
  constexpr int V = VecIO<T>::kVec;
  T const *X = static_cast<T const *>(x);
  T *Y = static_cast<T *>(y);
  if (inner == 1) {
    int ept = 0, wpr = 0;
    if (dim % V == 0 && aligned16(x) && aligned16(y) && pick_row_config(dim / V, ept, wpr)) {
      int64_t blocks = ceil_div(outer, 4 / wpr);
      bool const stream = stream_past_caches(outer * dim, sizeof(T));
#define CALL(E, W)                                                             \
  do {                                                                         \
    if (stream)                                                                \
      softmax_fwd_kernel<T, E, W, true><<<(unsigned)blocks, kRowThreads, 0, st>>>(X, Y, outer, (int)dim); \
    else                                                                       \
      softmax_fwd_kernel<T, E, W, false><<<(unsigned)blocks, kRowThreads, 0, st>>>(X, Y, outer, (int)dim); \
  } while (0)
      FFK_ROW_DISPATCH(ept, wpr, CALL);
#undef CALL
    } else {
      softmax_fwd_longrow_kernel<T><<<(unsigned)outer, kRowThreads, 0, st>>>(X, Y, dim);
    }
  } else {
    softmax_fwd_strided_kernel<T><<<(unsigned)ceil_div(outer * inner, 256), 256, 0, st>>>(
        X, Y, outer, dim, inner);
  }
  FFK_CHECK_LAUNCH();
  return FFK_OK;
}

template <typename T>
static int softmax_bwd(hipStream_t st, void const *y, void const *dy, void *dx,
                       int64_t outer, int64_t dim, int64_t inner) {
  constexpr int V = VecIO<T>::kVec;
  T const *Y = static_cast<T const *>(y);
  T const *DY = static_cast<T const *>(dy);
  T *DX = static_cast<T *>(dx);
  if (inner == 1) {
    int ept = 0, wpr = 0;
    if (dim % V == 0 && aligned16(y) && aligned16(dy) && aligned16(dx) &&
        pick_row_config(dim / V, ept, wpr)) {
      int64_t blocks = ceil_div(outer, 4 / wpr);
      bool const stream = stream_past_caches(outer * dim, sizeof(T));
#define CALL(E, W)                                                             \
  do {                                                                         \
    if (stream)                                                                \
      softmax_bwd_kernel<T, E, W, true><<<(unsigned)blocks, kRowThreads, 0, st>>>(Y, DY, DX, outer, (int)dim); \
    else                                                                       \
      softmax_bwd_kernel<T, E, W, false><<<(unsigned)blocks, kRowThreads, 0, st>>>(Y, DY, DX, outer, (int)dim); \
  } while (0)
      FFK_ROW_DISPATCH(ept, wpr, CALL);
#undef CALL
    } else {
      softmax_bwd_longrow_kernel<T><<<(unsigned)outer, kRowThreads, 0, st>>>(Y, DY, DX, dim);
    }
  } else {
    softmax_bwd_strided_kernel<T><<<(unsigned)ceil_div(outer * inner, 256), 256, 0, st>>>(
        Y, DY, DX, outer, dim, inner);
  }
  FFK_CHECK_LAUNCH();
  return FFK_OK;
}

}  // namespace ffk

using namespace ffk;

static int softmax_check(char const *who, int64_t outer, int64_t dim, int64_t inner) {
  FFK_REQUIRE(outer >= 0 && dim > 0 && inner > 0, "%s: bad shape", who);
  FFK_REQUIRE(dim < (1ll << 31), "%s: softmax dim too large", who);
  FFK_REQUIRE(outer * inner < (1ll << 31) * 256 && outer < (1ll << 31),
              "%s: too many rows", who);
  return FFK_OK;
}

extern "C" int ffk_softmax_forward(ffk_stream_t stream, int dtype,
                                   void const *input, void *output,
                                   int64_t outer, int64_t dim_size,
                                   int64_t inner) {
  int rc = softmax_check("softmax_forward", outer, dim_size, inner);
  if (rc != FFK_OK) return rc;
  if (outer == 0) return FFK_OK;
  FFK_REQUIRE(input && output, "softmax_forward: NULL tensor");
  if (dtype == FFK_FLOAT) return softmax_fwd<float>(as_stream(stream), input, output, outer, dim_size, inner);
  if (dtype == FFK_BF16) return softmax_fwd<bf16>(as_stream(stream), input, output, outer, dim_size, inner);
  return fail(FFK_ERR_UNSUPPORTED, "softmax_forward: dtype %d not supported", dtype);
}

extern "C" int ffk_softmax_backward(ffk_stream_t stream, int dtype,
                                    void const *output, void const *output_grad,
                                    void *input_grad, int64_t outer,
                                    int64_t dim_size, int64_t inner) {
  int rc = softmax_check("softmax_backward", outer, dim_size, inner);
  if (rc != FFK_OK) return rc;
  if (outer == 0) return FFK_OK;
  FFK_REQUIRE(output && output_grad && input_grad, "softmax_backward: NULL tensor");
  if (dtype == FFK_FLOAT) return softmax_bwd<float>(as_stream(stream), output, output_grad, input_grad, outer, dim_size, inner);
  if (dtype == FFK_BF16) return softmax_bwd<bf16>(as_stream(stream), output, output_grad, input_grad, outer, dim_size, inner);
  return fail(FFK_ERR_UNSUPPORTED, "softmax_backward: dtype %d not supported", dtype);
}

// The reference's backward: input_grad <- output_grad (softmax_kernels.cu:68-78).
extern "C" int ffk_softmax_backward_copy(ffk_stream_t stream, int dtype,
                                         void const *output_grad,
                                         void *input_grad,
                                         size_t num_elements) {
  size_t es = dtype_size(dtype);
  FFK_REQUIRE(es != 0, "softmax_backward_copy: bad dtype %d", dtype);
  if (num_elements == 0) return FFK_OK;
  FFK_REQUIRE(output_grad && input_grad, "softmax_backward_copy: NULL tensor");
  FFK_HIP(hipMemcpyAsync(input_grad, output_grad, num_elements * es,
                         hipMemcpyDeviceToDevice, as_stream(stream)));
  return FFK_OK;
}
