// Generic single-pass element-wise launcher: NIN inputs, NOUT outputs, all of
// element type T, arithmetic in fp32 through a functor.  Each lane moves
// 16 bytes per access and keeps kUnroll accesses in flight; a scalar tail (and
// a scalar path for unaligned pointers) keeps it correct for any length.
#pragma once
#include "ffk_common.h"

namespace ffk {

template <typename T, int NIN, int NOUT>
struct EwArgs {
  T const *in[NIN > 0 ? NIN : 1];
  int64_t in_elems[NIN > 0 ? NIN : 1];  // < n  =>  broadcast by index % elems
  T *out[NOUT];
  int64_t n;
};

// One 16-byte vector per lane and a grid that covers the tensor in one pass
// measured best on MI355X (deeper unrolling or a capped, looping grid lose 3-8%).
constexpr int kEwThreads = 256;
constexpr int kEwUnroll = 1;

template <typename T, int NIN, int NOUT, bool BCAST, typename F>
__global__ __launch_bounds__(kEwThreads) void ew_vec_kernel(
    EwArgs<T, NIN, NOUT> a, F f) {
  constexpr int V = VecIO<T>::kVec;
  int64_t const nvec = a.n / V;
  int64_t const stride = (int64_t)gridDim.x * kEwThreads;
  int64_t const step = stride * kEwUnroll;
  for (int64_t base = (int64_t)blockIdx.x * kEwThreads + threadIdx.x;
       base < nvec; base += step) {
    float x[kEwUnroll][NIN > 0 ? NIN : 1][V];
#pragma unroll
    for (int u = 0; u < kEwUnroll; u++) {
      int64_t i = base + u * stride;
      if (i < nvec) {
#pragma unroll
        for (int k = 0; k < NIN; k++) {
          int64_t off = i * V;
          if (BCAST) {
            off = off % a.in_elems[k];
          }
          // Measured on MI355X: with two or more input streams, loads that
          // bypass the caches lift a streaming kernel from ~70% to ~84% of HBM
          // peak; with a single input they cost ~8%.
          if (NIN >= 2 && !BCAST) {
            VecIO<T>::load_stream(a.in[k] + off, x[u][k]);
          } else {
            VecIO<T>::load(a.in[k] + off, x[u][k]);
          }
        }
      }
    }
#pragma unroll
    for (int u = 0; u < kEwUnroll; u++) {
      int64_t i = base + u * stride;
      if (i < nvec) {
        float y[NOUT][V];
#pragma unroll
        for (int e = 0; e < V; e++) {
          float xin[NIN > 0 ? NIN : 1];
          float yout[NOUT];
#pragma unroll
          for (int k = 0; k < NIN; k++) {
            xin[k] = x[u][k][e];
          }
          f(xin, yout);
#pragma unroll
          for (int k = 0; k < NOUT; k++) {
            y[k][e] = yout[k];
          }
        }
#pragma unroll
        for (int k = 0; k < NOUT; k++) {
          // one input fanned out to several outputs: streaming stores win
          if (NIN == 1 && NOUT >= 2) {
            VecIO<T>::store_stream(a.out[k] + i * V, y[k]);
          } else {
            VecIO<T>::store(a.out[k] + i * V, y[k]);
          }
        }
      }
    }
  }
  // scalar tail: the last n % V elements
  int64_t const t = nvec * V + (int64_t)blockIdx.x * kEwThreads + threadIdx.x;
  if (t < a.n) {
    float xin[NIN > 0 ? NIN : 1];
    float yout[NOUT];
#pragma unroll
    for (int k = 0; k < NIN; k++) {
      int64_t off = BCAST ? (t % a.in_elems[k]) : t;
      xin[k] = VecIO<T>::load1(a.in[k] + off);
    }
    f(xin, yout);
#pragma unroll
    for (int k = 0; k < NOUT; k++) {
      VecIO<T>::store1(a.out[k] + t, yout[k]);
    }
  }
}

template <typename T, int NIN, int NOUT, bool BCAST, typename F>
__global__ __launch_bounds__(kEwThreads) void ew_scalar_kernel(
    EwArgs<T, NIN, NOUT> a, F f) {
  int64_t const stride = (int64_t)gridDim.x * kEwThreads;
  for (int64_t t = (int64_t)blockIdx.x * kEwThreads + threadIdx.x; t < a.n;
       t += stride) {
    float xin[NIN > 0 ? NIN : 1];
    float yout[NOUT];
#pragma unroll
    for (int k = 0; k < NIN; k++) {
      int64_t off = BCAST ? (t % a.in_elems[k]) : t;
      xin[k] = VecIO<T>::load1(a.in[k] + off);
    }
    f(xin, yout);
#pragma unroll
    for (int k = 0; k < NOUT; k++) {
      VecIO<T>::store1(a.out[k] + t, yout[k]);
    }
  }
}

// Host launcher. Returns a hipError_t from the launch.
template <typename T, int NIN, int NOUT, typename F>
static inline hipError_t ew_launch(hipStream_t stream,
                                   EwArgs<T, NIN, NOUT> const &a, F f) {
  if (a.n <= 0) {
    return hipSuccess;
  }
  constexpr int V = VecIO<T>::kVec;
  bool vec_ok = true;
  bool bcast = false;
  for (int k = 0; k < NIN; k++) {
    vec_ok = vec_ok && aligned16(a.in[k]);
    if (a.in_elems[k] != a.n) {
      bcast = true;
      vec_ok = vec_ok && (a.in_elems[k] % V == 0);
    }
  }
  for (int k = 0; k < NOUT; k++) {
    vec_ok = vec_ok && aligned16(a.out[k]);
  }
  int64_t const max_blocks = (int64_t)1 << 30;
  if (vec_ok) {
    int64_t nvec = a.n / V;
    int64_t blocks = ceil_div(nvec > 0 ? nvec : 1, kEwThreads * kEwUnroll);
    if (blocks > max_blocks) {
      blocks = max_blocks;
    }
    if (bcast) {
      ew_vec_kernel<T, NIN, NOUT, true, F>
          <<<(int)blocks, kEwThreads, 0, stream>>>(a, f);
    } else {
      ew_vec_kernel<T, NIN, NOUT, false, F>
          <<<(int)blocks, kEwThreads, 0, stream>>>(a, f);
    }
  } else {
    int64_t blocks = ceil_div(a.n, kEwThreads);
    if (blocks > max_blocks) {
      blocks = max_blocks;
    }
    if (bcast) {
      ew_scalar_kernel<T, NIN, NOUT, true, F>
          <<<(int)blocks, kEwThreads, 0, stream>>>(a, f);
    } else {
      ew_scalar_kernel<T, NIN, NOUT, false, F>
          <<<(int)blocks, kEwThreads, 0, stream>>>(a, f);
    }
  }
  return hipGetLastError();
}

}  // namespace ffk
