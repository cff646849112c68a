// The dropout mask stream shared by the dropout kernels and the kernels that
// apply a dropout on the way (see dropout.hip for the definition of the
// stream: Philox4x32-10, one block per 8 elements, 16 bits per element).
#pragma once
#include "ffk_common.h"
#include <math.h>

namespace ffk {

struct PhiloxKey {
  uint32_t k0, k1;
};

__device__ __forceinline__ void philox4x32_10(uint64_t block, PhiloxKey key,
                                              uint32_t (&out)[4]) {
  uint32_t c0 = (uint32_t)block, c1 = (uint32_t)(block >> 32), c2 = 0u, c3 = 0u;
  uint32_t k0 = key.k0, k1 = key.k1;
#pragma unroll
  for (int r = 0; r < 10; r++) {
    uint64_t p0 = (uint64_t)0xD2511F53u * c0;
    uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
    uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
    uint32_t n1 = (uint32_t)p1;
    uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
    uint32_t n3 = (uint32_t)p0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

struct DropoutParams {
  PhiloxKey key;
  uint64_t offset;
  uint32_t threshold;  // keep iff the element's 16 bits >= threshold (0 .. 65536)
  float scale;         // 1 / (1 - rate)
};

// h: position of the element in its block of 8
__device__ __forceinline__ bool keep(uint32_t const (&w)[4], int h, DropoutParams const &p) {
  uint32_t const word = w[h >> 1];
  uint32_t const half = (h & 1) ? (word >> 16) : (word & 0xffffu);
  return half >= p.threshold;
}
__device__ __forceinline__ bool keep_dynamic(uint32_t const (&w)[4], uint32_t h, DropoutParams const &p) {
  uint32_t word = w[0];
  if ((h >> 1) == 1) word = w[1];
  if ((h >> 1) == 2) word = w[2];
  if ((h >> 1) == 3) word = w[3];
  uint32_t const half = (h & 1) ? (word >> 16) : (word & 0xffffu);
  return half >= p.threshold;
}

inline int make_dropout_params(char const *who, float rate, uint64_t seed,
                       uint64_t offset, DropoutParams &p) {
  FFK_REQUIRE(rate >= 0.0f && rate <= 1.0f, "%s: rate %f outside [0, 1]", who, (double)rate);
  p.threshold = (uint32_t)ceil((double)rate * 65536.0);  // 65536 (rate above 1 - 2^-16): everything dropped
  p.key.k0 = (uint32_t)seed;
  p.key.k1 = (uint32_t)(seed >> 32);
  p.offset = offset;
  p.scale = 1.0f / (1.0f - rate);
  return FFK_OK;
}

}  // namespace ffk
