// Measurement aid: what the matrix pipes of the whole chip deliver when nothing else limits them.
// One workgroup per CU, one wave per SIMD; every wave issues 32x32x16 bf16 MFMAs back to back on
// four independent accumulators, operands in registers, no memory access inside the loop.  The rate
// measured this way is the ceiling a GEMM kernel can approach on this card (its sustained clock
// under matrix load included), next to the vendor's 2.5 PFLOP/s figure for a fixed clock.
#include "ffk_common.h"

namespace ffk {

constexpr int kProbeMfmasPerIteration = 16;

__global__ __launch_bounds__(256) void mfma_probe_kernel(float *__restrict__ out, int iterations, uint32_t seed) {
  // operand bits from a hash of (lane, seed): values in [-1, 1), never NaN or infinite, so the
  // multipliers toggle like they do on real data (constant operands let the chip clock 15% higher)
  bf16x8 a, b;
  uint32_t h = (threadIdx.x + 1u) * 2654435761u ^ (seed * 40503u + 0x9e3779b9u);
#pragma unroll
  for (int i = 0; i < 8; i++) {
    h = h * 1664525u + 1013904223u;
    a[i] = (__bf16)((float)(int)(h >> 8 & 0xffff) * (1.0f / 32768.0f) - 1.0f);
    h = h * 1664525u + 1013904223u;
    b[i] = (__bf16)((float)(int)(h >> 8 & 0xffff) * (1.0f / 32768.0f) - 1.0f);
  }
  f32x16 acc[4];
#pragma unroll
  for (int j = 0; j < 4; j++) {
#pragma unroll
    for (int i = 0; i < 16; i++) acc[j][i] = 0.0f;
  }
  for (int it = 0; it < iterations; it++) {
#pragma unroll
    for (int j = 0; j < kProbeMfmasPerIteration; j++) {
      acc[j % 4] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[j % 4], 0, 0, 0);
    }
  }
  float s = 0.0f;
#pragma unroll
  for (int j = 0; j < 4; j++) {
#pragma unroll
    for (int i = 0; i < 16; i++) s += acc[j][i];
  }
  out[(size_t)blockIdx.x * 256 + threadIdx.x] = s;
}

}  // namespace ffk

using namespace ffk;

extern "C" int ffk_probe_mfma_bf16(ffk_stream_t stream, int iterations, uint32_t seed, float *out, size_t out_bytes,
                                   double *flops) {
  FFK_REQUIRE(iterations > 0 && iterations <= (1 << 20), "probe_mfma_bf16: 1 to 2^20 iterations, got %d", iterations);
  FFK_REQUIRE(out != nullptr && out_bytes >= (size_t)kNumCU * 256 * sizeof(float),
              "probe_mfma_bf16: out must hold %d floats", kNumCU * 256);
  mfma_probe_kernel<<<kNumCU, 256, 0, as_stream(stream)>>>(out, iterations, seed);
  FFK_CHECK_LAUNCH();
  // per wave and iteration: 16 MFMAs of 32 x 32 x 16 multiply-adds
  if (flops) *flops = (double)kNumCU * 4.0 * iterations * kProbeMfmasPerIteration * (2.0 * 32 * 32 * 16);
  return FFK_OK;
}
