// Shared device/host helpers for the gfx950 operator kernels: error reporting
// across the C ABI, bf16 <-> fp32 conversion, 16-byte vector access and
// wavefront (64-lane) reductions. Everything here is written for CDNA4 only.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include "../../include/ffk.h"

namespace ffk {

// ---- error plumbing -------------------------------------------------------
// Each entry point returns FFK_OK or an error code; the text is kept per
// thread and read back through ffk_last_error().
void set_error(char const *fmt, ...);
int fail(int code, char const *fmt, ...);
// current value of a process-wide switch (FFK_OPTION_*, see ffk_set_option)
int option(int which);

#define FFK_HIP(expr)                                                          \
  do {                                                                         \
    hipError_t e__ = (expr);                                                   \
    if (e__ != hipSuccess) {                                                   \
      return ::ffk::fail(FFK_ERR_HIP, "%s failed: %s (%s:%d)", #expr,          \
                         hipGetErrorString(e__), __FILE__, __LINE__);          \
    }                                                                          \
  } while (0)

#define FFK_REQUIRE(cond, ...)                                                 \
  do {                                                                         \
    if (!(cond)) {                                                             \
      return ::ffk::fail(FFK_ERR_INVALID, __VA_ARGS__);                        \
    }                                                                          \
  } while (0)

#define FFK_CHECK_LAUNCH() FFK_HIP(hipGetLastError())

static inline hipStream_t as_stream(ffk_stream_t s) {
  return reinterpret_cast<hipStream_t>(s);
}

static inline size_t dtype_size(int dt) {
  switch (dt) {
    case FFK_BOOL: return 1;
    case FFK_INT32: return 4;
    case FFK_INT64: return 8;
    case FFK_HALF: return 2;
    case FFK_FLOAT: return 4;
    case FFK_DOUBLE: return 8;
    case FFK_BF16: return 2;
    default: return 0;
  }
}

constexpr int kWave = 64;     // CDNA wavefront width
constexpr int kNumCU = 256;   // MI355X compute units (8 XCDs x 32)
constexpr int kNumXCD = 8;

// ---- bf16 -----------------------------------------------------------------
typedef __bf16 bf16;
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t bits16) {
  return __uint_as_float(bits16 << 16);
}
// Two fp32 -> packed bf16x2 in one instruction (v_cvt_pk_bf16_f32, RNE).
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  f32x2 v = {lo, hi};
  bf16x2 b = __builtin_convertvector(v, bf16x2);
  return __builtin_bit_cast(uint32_t, b);
}
// Round-to-nearest-even fp32 -> bf16 (the single rounding point of every
// bf16 kernel: inputs bf16 -> fp32 arithmetic -> one rounding at the store).
// The same hardware conversion as the packed stores, so a value rounded here
// and a value rounded by a vector store have the same bits, NaNs included.
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  return pack_bf16x2(f, 0.0f) & 0xffffu;
}

// ---- typed vector access: N elements of T <-> N floats --------------------
// VecIO<T>::kVec elements make one 16-byte access.
template <typename T>
struct VecIO;

template <>
struct VecIO<float> {
  static constexpr int kVec = 4;
  __device__ __forceinline__ static void load(float const *p, float (&v)[4]) {
    f32x4 r = *reinterpret_cast<f32x4 const *>(p);
    v[0] = r[0]; v[1] = r[1]; v[2] = r[2]; v[3] = r[3];
  }
  __device__ __forceinline__ static void store(float *p, float const (&v)[4]) {
    f32x4 r = {v[0], v[1], v[2], v[3]};
    *reinterpret_cast<f32x4 *>(p) = r;
  }
  // streaming variants: data touched once, do not keep it in the caches
  __device__ __forceinline__ static void load_stream(float const *p, float (&v)[4]) {
    f32x4 r = __builtin_nontemporal_load(reinterpret_cast<f32x4 const *>(p));
    v[0] = r[0]; v[1] = r[1]; v[2] = r[2]; v[3] = r[3];
  }
  __device__ __forceinline__ static void store_stream(float *p, float const (&v)[4]) {
    f32x4 r = {v[0], v[1], v[2], v[3]};
    __builtin_nontemporal_store(r, reinterpret_cast<f32x4 *>(p));
  }
  __device__ __forceinline__ static float load1(float const *p) { return *p; }
  __device__ __forceinline__ static void store1(float *p, float v) { *p = v; }
};

template <>
struct VecIO<bf16> {
  static constexpr int kVec = 8;
  __device__ __forceinline__ static void load(bf16 const *p, float (&v)[8]) {
    u32x4 r = *reinterpret_cast<u32x4 const *>(p);
#pragma unroll
    for (int i = 0; i < 4; i++) {
      v[2 * i] = __uint_as_float(r[i] << 16);
      v[2 * i + 1] = __uint_as_float(r[i] & 0xffff0000u);
    }
  }
  __device__ __forceinline__ static void store(bf16 *p, float const (&v)[8]) {
    u32x4 r;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      r[i] = pack_bf16x2(v[2 * i], v[2 * i + 1]);
    }
    *reinterpret_cast<u32x4 *>(p) = r;
  }
  __device__ __forceinline__ static void load_stream(bf16 const *p, float (&v)[8]) {
    u32x4 r = __builtin_nontemporal_load(reinterpret_cast<u32x4 const *>(p));
#pragma unroll
    for (int i = 0; i < 4; i++) {
      v[2 * i] = __uint_as_float(r[i] << 16);
      v[2 * i + 1] = __uint_as_float(r[i] & 0xffff0000u);
    }
  }
  __device__ __forceinline__ static void store_stream(bf16 *p, float const (&v)[8]) {
    u32x4 r;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      r[i] = pack_bf16x2(v[2 * i], v[2 * i + 1]);
    }
    __builtin_nontemporal_store(r, reinterpret_cast<u32x4 *>(p));
  }
  __device__ __forceinline__ static float load1(bf16 const *p) {
    return bf16_bits_to_f32(*reinterpret_cast<uint16_t const *>(p));
  }
  __device__ __forceinline__ static void store1(bf16 *p, float v) {
    *reinterpret_cast<uint16_t *>(p) = (uint16_t)f32_to_bf16_bits(v);
  }
};

// Raw 16-byte streaming load, unpacked later: lets a kernel issue the loads of
// its next row before it works on the current one.
__device__ __forceinline__ u32x4 load_raw_stream(void const *p) {
  return __builtin_nontemporal_load(reinterpret_cast<u32x4 const *>(p));
}
__device__ __forceinline__ void unpack_raw(u32x4 r, float (&v)[4], float const *) {
  v[0] = __uint_as_float(r[0]); v[1] = __uint_as_float(r[1]);
  v[2] = __uint_as_float(r[2]); v[3] = __uint_as_float(r[3]);
}
__device__ __forceinline__ void unpack_raw(u32x4 r, float (&v)[8], bf16 const *) {
#pragma unroll
  for (int i = 0; i < 4; i++) {
    v[2 * i] = __uint_as_float(r[i] << 16);
    v[2 * i + 1] = __uint_as_float(r[i] & 0xffff0000u);
  }
}

// ---- GELU (exact erf form) shared by ElementUnary and the GEMM epilogue ----
// erf by Abramowitz & Stegun 7.1.26 (|error| <= 1.5e-7), sharing exp(-z^2)
// with the caller: returns erf(z) given e = exp(-z*z).
__device__ __forceinline__ float erf_from_exp(float z, float e) {
  float const az = fabsf(z);
  // v_rcp_f32 (1 ulp) instead of an IEEE division: the polynomial's own error is 1.5e-7
  float const t = __builtin_amdgcn_rcpf(1.0f + 0.3275911f * az);
  float poly = 1.061405429f;
  poly = poly * t - 1.453152027f;
  poly = poly * t + 1.421413741f;
  poly = poly * t - 0.284496736f;
  poly = poly * t + 0.254829592f;
  float const r = 1.0f - poly * t * e;
  return copysignf(r, z);
}
// x/2 erfc(-x/sqrt2) = x (1/2 + 1/2 erf(x/sqrt2))
__device__ __forceinline__ float gelu_forward(float v) {
  float const z = v * 0.70710678118654752440f;
  return v * (0.5f + 0.5f * erf_from_exp(z, __expf(-z * z)));
}

// d/dx [x Phi(x)] = Phi(x) + x phi(x)
__device__ __forceinline__ float gelu_derivative(float x) {
  float const z = x * 0.70710678118654752440f;
  float const e = __expf(-z * z);  // = exp(-x^2 / 2), shared by Phi and phi
  return 0.5f + 0.5f * erf_from_exp(z, e) + x * 0.39894228040143267794f * e;
}

// Value a float takes after a round trip through the storage type: what a
// following op would read had this value been stored in between.
template <typename T>
__device__ __forceinline__ float storage_round(float v);
template <>
__device__ __forceinline__ float storage_round<float>(float v) { return v; }
template <>
__device__ __forceinline__ float storage_round<bf16>(float v) {
  return __uint_as_float(pack_bf16x2(v, 0.0f) << 16);
}

// ---- wavefront reductions (64 lanes) ---------------------------------------
// Every lane ends with the result over all 64.  The first four steps read the partner lane
// through the vector ALU's own lane-select (DPP) and the last two through the 16- and 32-lane
// swaps: eight vector instructions and no trip through the LDS crossbar, which a shuffle-based
// butterfly (ds_bpermute) pays six times in a row, each with an LDS round trip of latency.
//   quad_perm [1,0,3,2], quad_perm [2,3,0,1]: partners 1 and 2 lanes away (all 4 of a quad equal);
//   row_half_mirror: lane i of 8 reads lane 7 - i, which lies in the other quad;
//   row_mirror: lane i of 16 reads lane 15 - i, which lies in the other group of 8.
// Partners always apply the commutative operation to the same two values, so the lanes agree
// bit for bit.
template <int CTRL>
__device__ __forceinline__ float dpp_read(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
template <typename F>
__device__ __forceinline__ float wave_reduce(float v, F f) {
  v = f(v, dpp_read<0xB1>(v));   // quad_perm [1,0,3,2]
  v = f(v, dpp_read<0x4E>(v));   // quad_perm [2,3,0,1]
  v = f(v, dpp_read<0x141>(v));  // row_half_mirror
  v = f(v, dpp_read<0x140>(v));  // row_mirror
  // swaps the odd 16-lane rows of the first operand with the even rows of the second: with the
  // same value in both, the results hold rows {0,0,2,2} and {1,1,3,3}
  auto const a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = f(__uint_as_float(a[0]), __uint_as_float(a[1]));
  // the same for the two 32-lane halves
  auto const b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return f(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float wave_sum(float v) {
  return wave_reduce(v, [](float a, float b) { return a + b; });
}
__device__ __forceinline__ float wave_max(float v) {
  return wave_reduce(v, [](float a, float b) { return fmaxf(a, b); });
}

// ---- division by a number fixed at launch ---------------------------------
// The compiler expands an integer division by a kernel argument into some 40 (32-bit) to 130
// (64-bit) instructions, which is what a thread that moves 16 or 32 bytes can least afford.
// For n < 2^31 and 1 <= d < 2^31: with L = ceil(log2 d), k = 31 + L and M = ceil(2^k / d)
// (M <= 2^32 - 1 for d >= 2; d = 1 is a shift by zero of n itself), floor(n M / 2^k) = floor(n / d),
// because the excess M d - 2^k is below 2^L and n times it stays below 2^k.
struct FastDiv {
  uint32_t mul;
  uint32_t shift;
  uint32_t d;
  __device__ __forceinline__ uint32_t div(uint32_t n) const {
    return d == 1 ? n : (uint32_t)(((uint64_t)n * mul) >> shift);
  }
  // quotient and remainder
  __device__ __forceinline__ void divmod(uint32_t n, uint32_t &q, uint32_t &r) const {
    q = div(n);
    r = n - q * d;
  }
};
static inline FastDiv make_fast_div(uint32_t d) {
  FastDiv f;
  f.d = d;
  uint32_t L = 0;
  while (((uint64_t)1 << L) < d) L++;
  f.shift = 31 + L;
  f.mul = d <= 1 ? 0u : (uint32_t)((((uint64_t)1 << f.shift) + d - 1) / d);
  return f;
}

// A tensor this large does not stay in the 256 MB last-level cache between the kernel that
// writes it and the one that reads it next: its accesses then bypass the caches (non-temporal
// loads and stores), which measured 6-8% more bandwidth on 1 GB softmax tensors.  Smaller
// tensors keep ordinary accesses so the next kernel finds them in cache.
static inline bool stream_past_caches(int64_t elems, size_t elem_size) {
  return (size_t)elems * elem_size > ((size_t)128 << 20);
}

// A kernel that uses more than 64 KB of dynamic LDS has to be given leave, once on every device
// it is launched on (the attribute belongs to the device's copy of the code).  One object per
// kernel instantiation; ensure() costs a hipGetDevice per launch after the first.  Concurrent
// first calls may both set the attribute, which is harmless.
struct LdsOptIn {
  static constexpr int kMaxDevices = 64;
  bool done[kMaxDevices] = {};
  hipError_t ensure(void const *kernel, int bytes) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    bool const tracked = dev >= 0 && dev < kMaxDevices;
    if (tracked && done[dev]) return hipSuccess;
    e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e == hipSuccess && tracked) done[dev] = true;
    return e;
  }
};

static inline bool aligned16(void const *p) {
  return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}

__host__ __device__ static inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

}  // namespace ffk
