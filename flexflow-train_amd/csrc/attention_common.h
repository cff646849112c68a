// Pieces shared by the bf16 attention kernels: the parameter blocks of the
// forward and backward kernels and the LDS fragment readers for the 32x32x16 bf16 MFMA.
#pragma once
#include "ffk_common.h"
#include <type_traits>

namespace ffk {

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

typedef s16x4 __attribute__((address_space(3))) * lds_s16x4_ptr;

struct AttnParams {
  bf16 const *q, *k, *v;
  bf16 *o;
  float *lse;
  int B, H, Sq, Skv;
  int64_t q_bs, q_ss, k_bs, k_ss, v_bs, v_ss, o_bs, o_ss;
  float scale_log2;  // scale * log2(e)
  int causal;
};

struct AttnBwdParams {
  bf16 const *q, *k, *v, *o, *d_o;
  float const *lse;
  float *delta;
  bf16 *dq, *dk, *dv;
  int B, H, Sq, Skv;
  int64_t q_bs, q_ss, k_bs, k_ss, v_bs, v_ss, o_bs, o_ss;
  float scale, scale_log2;
  int causal;
};

__device__ __forceinline__ bf16x8 pack8(float const *v) {
  union {
    uint32_t u[4];
    bf16x8 b;
  } x;
#pragma unroll
  for (int i = 0; i < 4; i++) x.u[i] = pack_bf16x2(v[2 * i], v[2 * i + 1]);
  return x.b;
}

// B- or A-operand fragment from a row-major LDS tile whose rows are the
// operand's rows/columns and whose contiguous dim is the reduction dim.
// The lane-dependent part of the address (lane_k_off) is computed once per
// kernel; row0 / k0 are compile-time after unrolling and fold into the
// instruction's offset field.
__device__ __forceinline__ int lane_k_off(int stride, int lane) {
  return (lane & 31) * stride + (lane >> 5) * 8;
}
__device__ __forceinline__ bf16x8 frag_k(bf16 const *tile_plus_lane, int stride,
                                         int row0, int k0) {
  return *reinterpret_cast<bf16x8 const *>(tile_plus_lane + row0 * stride + k0);
}

// Fragment from an LDS tile stored [reduction index][row/column index]
// (contiguous along the operand's non-reduction dim), using the reduction
// order of an accumulator re-used as the other operand: k-slot (h, j) of step
// s is tile row  r0 + 16 s + 8 (j / 4) + 4 h + j % 4.
__device__ __forceinline__ int lane_tr_off(int stride, int lane) {
  int const i16 = lane & 15;
  return (4 * (lane >> 5) + (i16 >> 2)) * stride + ((lane >> 4) & 1) * 16 + (i16 & 3) * 4;
}
__device__ __forceinline__ bf16x8 frag_tr_acc(bf16 const *tile_plus_lane, int stride,
                                              int r0, int s, int col0) {
  bf16 const *p = tile_plus_lane + (r0 + 16 * s) * stride + col0;
  s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p));
  s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p + 8 * stride));
  union {
    s16x4 h2[2];
    bf16x8 v;
  } u;
  u.h2[0] = lo;
  u.h2[1] = hi;
  return u.v;
}

// Compile-time loop: f(std::integral_constant<int, I>) for I = 0 .. N-1.
template <int I, int N, typename F>
__device__ __forceinline__ void static_for(F &&f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<I + 1, N>(f);
  }
}

// Ties a value to this point of the program: the arithmetic that produces it cannot be moved
// behind it by the optimizer (which otherwise gathers a unit of vector work placed between two
// MFMAs at the place where its result is first needed).
__device__ __forceinline__ void pin_here(float &x) { asm volatile("" : "+v"(x)); }

// Maximum of a value over the two lanes l and l ^ 32 (they hold the same query's column).
__device__ __forceinline__ float max_across_halves(float x) {
  // swaps the upper 32 lanes of the first operand with the lower 32 of the second: with the same
  // value in both, one result holds the lower half twice and the other the upper half twice
  auto const r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}


}  // namespace ffk
