// Row-wise reduction scaffolding shared by LayerNorm and Softmax.
//
// A row of N elements is owned either by one wavefront (WPR == 1: no LDS, no
// barrier, four independent rows per 256-thread workgroup) or by the four
// wavefronts of a workgroup (WPR == 4).  Each lane keeps EPT 16-byte vectors
// of the row in registers, so every element is read from HBM exactly once.
#pragma once
#include "ffk_common.h"

namespace ffk {

constexpr int kRowThreads = 256;

template <int WPR>
struct RowReducer {
  // smem: 2 phases x 4 waves x 2 values
  float (*smem)[4][2];
  int phase;
  __device__ __forceinline__ RowReducer(float (*s)[4][2]) : smem(s), phase(0) {}

  __device__ __forceinline__ void sum2(float &a, float &b) {
    a = wave_sum(a);
    b = wave_sum(b);
    if (WPR > 1) {
      int const wave = threadIdx.x >> 6;
      if ((threadIdx.x & 63) == 0) {
        smem[phase][wave][0] = a;
        smem[phase][wave][1] = b;
      }
      __syncthreads();
      a = smem[phase][0][0] + smem[phase][1][0] + smem[phase][2][0] + smem[phase][3][0];
      b = smem[phase][0][1] + smem[phase][1][1] + smem[phase][2][1] + smem[phase][3][1];
      phase ^= 1;
    }
  }
  __device__ __forceinline__ float sum(float a) {
    float b = 0.0f;
    sum2(a, b);
    return a;
  }
  __device__ __forceinline__ float max(float a) {
    a = wave_max(a);
    if (WPR > 1) {
      int const wave = threadIdx.x >> 6;
      if ((threadIdx.x & 63) == 0) {
        smem[phase][wave][0] = a;
      }
      __syncthreads();
      a = fmaxf(fmaxf(smem[phase][0][0], smem[phase][1][0]),
                fmaxf(smem[phase][2][0], smem[phase][3][0]));
      phase ^= 1;
    }
    return a;
  }
};

// Picks (EPT, WPR) for a row of `nvec` 16-byte vectors; returns false when the
// row does not fit in registers (nvec > 256 * 8).
static inline bool pick_row_config(int64_t nvec, int &ept, int &wpr) {
  if (nvec <= 64 * 8) {
    wpr = 1;
    ept = nvec <= 64 ? 1 : nvec <= 128 ? 2 : nvec <= 256 ? 4 : 8;
    return true;
  }
  if (nvec <= 256 * 8) {
    wpr = 4;
    ept = nvec <= 256 * 4 ? 4 : 8;
    return true;
  }
  return false;
}

// Row configuration used by the kernels: one wave per row up to 128 vectors,
// one workgroup per row beyond (few vectors per lane keeps register use low and
// measured 76% vs 59% of HBM peak for a [16384, 4096] bf16 LayerNorm forward).
static inline bool pick_row_config_small(int64_t nvec, int &ept, int &wpr) {
  if (nvec <= 128) {
    wpr = 1;
    ept = nvec <= 64 ? 1 : 2;
    return true;
  }
  if (nvec <= 256 * 8) {
    wpr = 4;
    ept = nvec <= 256 ? 1 : nvec <= 512 ? 2 : nvec <= 1024 ? 4 : 8;
    return true;
  }
  return false;
}

#define FFK_ROW_DISPATCH_SMALL(EPT_, WPR_, CALL)                               \
  do {                                                                         \
    if ((WPR_) == 1) {                                                         \
      if ((EPT_) == 1) { CALL(1, 1); }                                         \
      else { CALL(2, 1); }                                                     \
    } else {                                                                   \
      if ((EPT_) == 1) { CALL(1, 4); }                                         \
      else if ((EPT_) == 2) { CALL(2, 4); }                                    \
      else if ((EPT_) == 4) { CALL(4, 4); }                                    \
      else { CALL(8, 4); }                                                     \
    }                                                                          \
  } while (0)

#define FFK_ROW_DISPATCH(EPT_, WPR_, CALL)                                     \
  do {                                                                         \
    if ((WPR_) == 1) {                                                         \
      if ((EPT_) == 1) { CALL(1, 1); }                                         \
      else if ((EPT_) == 2) { CALL(2, 1); }                                    \
      else if ((EPT_) == 4) { CALL(4, 1); }                                    \
      else { CALL(8, 1); }                                                     \
    } else {                                                                   \
      if ((EPT_) == 4) { CALL(4, 4); }                                         \
      else { CALL(8, 4); }                                                     \
    }                                                                          \
  } while (0)

}  // namespace ffk
