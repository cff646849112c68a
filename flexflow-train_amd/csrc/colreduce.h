// Column sums of an fp32 partials matrix [nparts][ncols] -- the second pass of
// the bias-gradient (column-sum) and LayerNorm gamma/beta-gradient reductions.
// A workgroup of 1024 threads owns 32 columns; its 32 row groups read the
// partial rows in parallel (every load an independent 128-byte segment, up to
// four in flight per thread) and meet in LDS, so a few hundred partial rows
// cost one or two memory round trips instead of a serial walk.
#pragma once
#include "ffk_common.h"

namespace ffk {

// Columns [0, split) go to out0, columns [split, ncols) to out1 (either may be
// NULL: that half is skipped).  accumulate adds the old output value.
template <typename T>
__global__ __launch_bounds__(1024) void colreduce_kernel(
    float const *__restrict__ partials, int nparts, int ncols, int split,
    T *out0, T *out1, int accumulate) {
  __shared__ float red[32][33];
  int const cx = threadIdx.x & 31, ry = threadIdx.x >> 5;
  int const j = blockIdx.x * 32 + cx;
  float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f, s3 = 0.0f;
  if (j < ncols) {
    float const *p = partials + j;
    int r = ry;
    for (; r + 96 < nparts; r += 128) {
      s0 += p[(int64_t)r * ncols];
      s1 += p[(int64_t)(r + 32) * ncols];
      s2 += p[(int64_t)(r + 64) * ncols];
      s3 += p[(int64_t)(r + 96) * ncols];
    }
    for (; r < nparts; r += 32) s0 += p[(int64_t)r * ncols];
  }
  red[ry][cx] = (s0 + s1) + (s2 + s3);
  __syncthreads();
  if (ry == 0 && j < ncols) {
    float t = 0.0f;
#pragma unroll
    for (int r = 0; r < 32; r++) t += red[r][cx];
    T *out = j < split ? out0 : out1;
    int const jo = j < split ? j : j - split;
    if (out != nullptr) {
      if (accumulate) t += VecIO<T>::load1(out + jo);
      VecIO<T>::store1(out + jo, t);
    }
  }
}

template <typename T>
inline hipError_t colreduce_launch(hipStream_t st, float const *partials,
                                   int nparts, int ncols, int split, T *out0,
                                   T *out1, bool accumulate) {
  colreduce_kernel<T><<<(unsigned)ceil_div(ncols, 32), 1024, 0, st>>>(
      partials, nparts, ncols, split, out0, out1, accumulate ? 1 : 0);
  return hipGetLastError();
}

}  // namespace ffk
