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
struct ColreduceJob {
  float const *partials;
  int nparts, ncols, split;
  void *out0, *out1;
  int accumulate;
};

template <typename T>
__device__ __forceinline__ void colreduce_block(ColreduceJob const &job, int block, float (&red)[32][33]) {
  int const cx = threadIdx.x & 31, ry = threadIdx.x >> 5;
  int const j = block * 32 + cx;
  float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f, s3 = 0.0f;
  if (j < job.ncols) {
    float const *p = job.partials + j;
    int r = ry;
    for (; r + 96 < job.nparts; r += 128) {
      s0 += p[(int64_t)r * job.ncols];
      s1 += p[(int64_t)(r + 32) * job.ncols];
      s2 += p[(int64_t)(r + 64) * job.ncols];
      s3 += p[(int64_t)(r + 96) * job.ncols];
    }
    for (; r < job.nparts; r += 32) s0 += p[(int64_t)r * job.ncols];
  }
  red[ry][cx] = (s0 + s1) + (s2 + s3);
  __syncthreads();
  if (ry == 0 && j < job.ncols) {
    float t = 0.0f;
#pragma unroll
    for (int r = 0; r < 32; r++) t += red[r][cx];
    T *out = static_cast<T *>(j < job.split ? job.out0 : job.out1);
    int const jo = j < job.split ? j : j - job.split;
    if (out != nullptr) {
      if (job.accumulate) t += VecIO<T>::load1(out + jo);
      VecIO<T>::store1(out + jo, t);
    }
  }
}

template <typename T>
__global__ __launch_bounds__(1024) void colreduce_kernel(ColreduceJob job) {
  __shared__ float red[32][33];
  colreduce_block<T>(job, (int)blockIdx.x, red);
}

// Several reductions in one launch: a caller that runs a sequence of operators
// whose column sums are only needed at the end (the bias and LayerNorm
// parameter gradients of a layer's backward pass) collects them instead of
// paying one tiny launch each.  Each job keeps its own partials until the
// flush, so the producers must not share scratch.
constexpr int kMaxColreduceJobs = 8;
struct ColreduceBatch {
  ColreduceJob job[kMaxColreduceJobs];
  int first_block[kMaxColreduceJobs + 1];
  int count = 0;
  int dtype = -1;
};
// non-null while a caller on this thread is collecting
inline thread_local ColreduceBatch *tl_colreduce_batch = nullptr;

template <typename T>
__global__ __launch_bounds__(1024) void colreduce_batch_kernel(ColreduceBatch b) {
  __shared__ float red[32][33];
  int k = 0;
  while (k + 1 < b.count && (int)blockIdx.x >= b.first_block[k + 1]) k++;
  colreduce_block<T>(b.job[k], (int)blockIdx.x - b.first_block[k], red);
}

// Runs what was collected (nothing to do for an empty batch) and empties it.
inline hipError_t colreduce_flush(hipStream_t st, ColreduceBatch &b) {
  if (b.count == 0) return hipSuccess;
  int const blocks = b.first_block[b.count - 1] + (int)ceil_div(b.job[b.count - 1].ncols, 32);
  b.first_block[b.count] = blocks;
  if (b.dtype == FFK_FLOAT) {
    colreduce_batch_kernel<float><<<(unsigned)blocks, 1024, 0, st>>>(b);
  } else {
    colreduce_batch_kernel<bf16><<<(unsigned)blocks, 1024, 0, st>>>(b);
  }
  b.count = 0;
  return hipGetLastError();
}

template <typename T>
inline hipError_t colreduce_launch(hipStream_t st, float const *partials,
                                   int nparts, int ncols, int split, T *out0,
                                   T *out1, bool accumulate) {
  ColreduceJob const job{partials, nparts, ncols, split, out0, out1, accumulate ? 1 : 0};
  ColreduceBatch *b = tl_colreduce_batch;
  int const dtype = sizeof(T) == 4 ? FFK_FLOAT : FFK_BF16;
  if (b != nullptr) {
    // The collected jobs run as one launch, in no order: a job that writes where a collected
    // one writes (a bias shared by two Linear layers) would race with it.  Run what is
    // collected first; this job then follows it on the stream.
    for (int k = 0; k < b->count; k++) {
      ColreduceJob const &c = b->job[k];
      bool const clash = (out0 != nullptr && (c.out0 == out0 || c.out1 == out0)) ||
                         (out1 != nullptr && (c.out0 == out1 || c.out1 == out1));
      if (clash) {
        hipError_t e = colreduce_flush(st, *b);
        if (e != hipSuccess) return e;
        break;
      }
    }
  }
  if (b != nullptr && b->count < kMaxColreduceJobs && (b->count == 0 || b->dtype == dtype)) {
    b->first_block[b->count] = b->count == 0 ? 0 : b->first_block[b->count - 1] + (int)ceil_div(b->job[b->count - 1].ncols, 32);
    b->job[b->count] = job;
    b->dtype = dtype;
    b->count++;
    return hipSuccess;
  }
  colreduce_kernel<T><<<(unsigned)ceil_div(ncols, 32), 1024, 0, st>>>(job);
  return hipGetLastError();
}

}  // namespace ffk
