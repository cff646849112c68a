// Cast forward/backward for gfx950 (reference: lib/kernels/src/cuda/ops/
// cast_kernels.cu:25-37, CPU lib/kernels/src/kernels/cast_kernels_cpu.cc).
//   forward : output[i] = (ODT) input[i]
//   backward: input_grad[i] = (ODT) output_grad[i] + 1 * input_grad[i]
// Any pair of {bool, int32, int64, half, float, double, bf16}; conversions follow
// C++ static_cast except float -> bf16/half, which round to nearest even.
#include "ffk_common.h"
#include <type_traits>

namespace ffk {

constexpr int kCastThreads = 256;

template <typename T> struct IsBf16 { static constexpr bool value = false; };
template <> struct IsBf16<bf16> { static constexpr bool value = true; };
template <typename T> struct IsBool { static constexpr bool value = false; };
template <> struct IsBool<bool> { static constexpr bool value = true; };
template <typename T> struct IsHalf { static constexpr bool value = false; };
template <> struct IsHalf<_Float16> { static constexpr bool value = true; };

// static_cast<ODT>(x) with bf16 handled through its fp32 value (round to
// nearest even on the way in) and bool as "non-zero".
template <typename ODT, typename IDT>
__device__ __forceinline__ ODT convert(IDT x) {
  if constexpr (IsBf16<IDT>::value) {
    float const f = bf16_bits_to_f32(*reinterpret_cast<uint16_t const *>(&x));
    return convert<ODT, float>(f);
  } else if constexpr (IsBf16<ODT>::value) {
    float f;
    if constexpr (IsBool<IDT>::value) f = x ? 1.0f : 0.0f;
    else f = static_cast<float>(x);
    uint16_t const bits = (uint16_t)f32_to_bf16_bits(f);
    return *reinterpret_cast<bf16 const *>(&bits);
  } else if constexpr (IsBool<ODT>::value) {
    return x != static_cast<IDT>(0);
  } else if constexpr (IsBool<IDT>::value) {
    return static_cast<ODT>(x ? 1 : 0);
  } else if constexpr (IsHalf<IDT>::value || IsHalf<ODT>::value) {
    return static_cast<ODT>(static_cast<float>(x));
  } else {
    return static_cast<ODT>(x);
  }
}

// a + b in the type's own arithmetic (bf16/half: add in fp32, round once;
// bool: logical or, as `bool + 1 * bool` converts back to bool)
template <typename T>
__device__ __forceinline__ T add_in_type(T a, T b) {
  if constexpr (IsBf16<T>::value) {
    return convert<T, float>(convert<float, T>(a) + convert<float, T>(b));
  } else if constexpr (IsHalf<T>::value) {
    return static_cast<T>(static_cast<float>(a) + static_cast<float>(b));
  } else if constexpr (IsBool<T>::value) {
    return a || b;
  } else {
    return static_cast<T>(a + b);
  }
}

template <typename IDT, typename ODT, bool BACKWARD>
__global__ __launch_bounds__(kCastThreads) void cast_kernel(IDT const *__restrict__ in, ODT *out, int64_t n) {
  int64_t const stride = (int64_t)gridDim.x * kCastThreads;
  for (int64_t i = (int64_t)blockIdx.x * kCastThreads + threadIdx.x; i < n; i += stride) {
    ODT c = convert<ODT, IDT>(in[i]);
    if (BACKWARD) c = add_in_type<ODT>(c, out[i]);
    out[i] = c;
  }
}

// V consecutive elements moved as one naturally aligned object, so a lane's
// loads and stores are 16-byte (or, for the narrower side, 8- or 4-byte) accesses
template <typename T, int V>
struct alignas(sizeof(T) * V > 16 ? 16 : sizeof(T) * V) CastPack {
  T v[V];
};

template <typename IDT, typename ODT>
constexpr int cast_pack_width() {
  return (sizeof(IDT) > 4 || sizeof(ODT) > 4) ? 4 : 8;
}

// A pack moved in its widest aligned units (16, 8 or 4 bytes); STREAM: past the caches, for
// tensors that neither fit them nor are read again soon.
template <typename P>
struct PackUnit {
  using type = std::conditional_t<sizeof(P) >= 16, u32x4, std::conditional_t<sizeof(P) == 8, uint64_t, uint32_t>>;
  static_assert(sizeof(P) % sizeof(type) == 0 && alignof(P) >= (sizeof(P) >= 16 ? 16 : sizeof(P)), "pack layout");
};
template <bool STREAM, typename P>
__device__ __forceinline__ P load_pack(P const *p) {
  using U = typename PackUnit<P>::type;
  union {
    P pack;
    U u[sizeof(P) / sizeof(U)];
  } x;
#pragma unroll
  for (unsigned i = 0; i < sizeof(P) / sizeof(U); i++) {
    U const *src = reinterpret_cast<U const *>(p) + i;
    x.u[i] = STREAM ? __builtin_nontemporal_load(src) : *src;
  }
  return x.pack;
}
template <bool STREAM, typename P>
__device__ __forceinline__ void store_pack(P *p, P const &v) {
  using U = typename PackUnit<P>::type;
  union {
    P pack;
    U u[sizeof(P) / sizeof(U)];
  } x;
  x.pack = v;
#pragma unroll
  for (unsigned i = 0; i < sizeof(P) / sizeof(U); i++) {
    U *dst = reinterpret_cast<U *>(p) + i;
    if (STREAM) {
      __builtin_nontemporal_store(x.u[i], dst);
    } else {
      *dst = x.u[i];
    }
  }
}

// Two packs per thread and iteration: all loads of both are issued before the first conversion.
template <typename IDT, typename ODT, bool BACKWARD, bool STREAM>
__global__ __launch_bounds__(kCastThreads) void cast_vec_kernel(IDT const *__restrict__ in, ODT *out, int64_t n) {
  constexpr int V = cast_pack_width<IDT, ODT>();
  using PI = CastPack<IDT, V>;
  using PO = CastPack<ODT, V>;
  int64_t const packs = n / V;
  int64_t const stride = (int64_t)gridDim.x * kCastThreads;
  int64_t const tid = (int64_t)blockIdx.x * kCastThreads + threadIdx.x;
  PI const *pin = reinterpret_cast<PI const *>(in);
  PO *pout = reinterpret_cast<PO *>(out);
  auto convert_pack = [](PI const &a, PO &o) {
#pragma unroll
    for (int e = 0; e < V; e++) {
      ODT c = convert<ODT, IDT>(a.v[e]);
      if (BACKWARD) c = add_in_type<ODT>(c, o.v[e]);
      o.v[e] = c;
    }
  };
  int64_t p = tid;
  for (; p + stride < packs; p += 2 * stride) {
    PI const a0 = load_pack<STREAM>(pin + p), a1 = load_pack<STREAM>(pin + p + stride);
    PO o0, o1;
    if (BACKWARD) {
      o0 = load_pack<STREAM>(pout + p);
      o1 = load_pack<STREAM>(pout + p + stride);
    }
    convert_pack(a0, o0);
    convert_pack(a1, o1);
    store_pack<STREAM>(pout + p, o0);
    store_pack<STREAM>(pout + p + stride, o1);
  }
  if (p < packs) {
    PI const a = load_pack<STREAM>(pin + p);
    PO o;
    if (BACKWARD) o = load_pack<STREAM>(pout + p);
    convert_pack(a, o);
    store_pack<STREAM>(pout + p, o);
  }
  int64_t const j = packs * V + tid;
  if (j < n) {
    ODT c = convert<ODT, IDT>(in[j]);
    if (BACKWARD) c = add_in_type<ODT>(c, out[j]);
    out[j] = c;
  }
}

template <typename IDT, typename ODT>
static hipError_t cast_launch(hipStream_t st, void const *in, void *out, int64_t n, bool backward) {
  constexpr int V = cast_pack_width<IDT, ODT>();
  bool const vec = n >= V && reinterpret_cast<uintptr_t>(in) % alignof(CastPack<IDT, V>) == 0 &&
                   reinterpret_cast<uintptr_t>(out) % alignof(CastPack<ODT, V>) == 0;
  int64_t b = ceil_div(vec ? n / V : n, kCastThreads);
  int64_t const cap = (int64_t)kNumCU * 64;
  unsigned const blocks = (unsigned)(b < cap ? b : cap);
  IDT const *ip = static_cast<IDT const *>(in);
  ODT *op = static_cast<ODT *>(out);
  if (vec) {
    // input and output together beyond half the last-level cache: move them past the caches
    bool const stream = (double)n * (sizeof(IDT) + sizeof(ODT)) > 128.0 * 1024 * 1024;
    if (backward) {
      if (stream) cast_vec_kernel<IDT, ODT, true, true><<<blocks, kCastThreads, 0, st>>>(ip, op, n);
      else cast_vec_kernel<IDT, ODT, true, false><<<blocks, kCastThreads, 0, st>>>(ip, op, n);
    } else {
      if (stream) cast_vec_kernel<IDT, ODT, false, true><<<blocks, kCastThreads, 0, st>>>(ip, op, n);
      else cast_vec_kernel<IDT, ODT, false, false><<<blocks, kCastThreads, 0, st>>>(ip, op, n);
    }
  } else {
    if (backward) cast_kernel<IDT, ODT, true><<<blocks, kCastThreads, 0, st>>>(ip, op, n);
    else cast_kernel<IDT, ODT, false><<<blocks, kCastThreads, 0, st>>>(ip, op, n);
  }
  return hipGetLastError();
}

template <typename IDT>
static int cast_out(char const *who, hipStream_t st, int out_dtype, void const *in, void *out,
                    int64_t n, bool backward) {
  hipError_t e;
  switch (out_dtype) {
    case FFK_BOOL: e = cast_launch<IDT, bool>(st, in, out, n, backward); break;
    case FFK_INT32: e = cast_launch<IDT, int32_t>(st, in, out, n, backward); break;
    case FFK_INT64: e = cast_launch<IDT, int64_t>(st, in, out, n, backward); break;
    case FFK_HALF: e = cast_launch<IDT, _Float16>(st, in, out, n, backward); break;
    case FFK_FLOAT: e = cast_launch<IDT, float>(st, in, out, n, backward); break;
    case FFK_DOUBLE: e = cast_launch<IDT, double>(st, in, out, n, backward); break;
    case FFK_BF16: e = cast_launch<IDT, bf16>(st, in, out, n, backward); break;
    default: return fail(FFK_ERR_UNSUPPORTED, "%s: output dtype %d not supported", who, out_dtype);
  }
  FFK_HIP(e);
  return FFK_OK;
}

static int cast_any(char const *who, ffk_stream_t stream, int in_dtype, int out_dtype,
                    void const *in, void *out, int64_t n, bool backward) {
  FFK_REQUIRE(n >= 0, "%s: negative size", who);
  if (n == 0) return FFK_OK;
  FFK_REQUIRE(in && out, "%s: NULL tensor", who);
  hipStream_t st = as_stream(stream);
  switch (in_dtype) {
    case FFK_BOOL: return cast_out<bool>(who, st, out_dtype, in, out, n, backward);
    case FFK_INT32: return cast_out<int32_t>(who, st, out_dtype, in, out, n, backward);
    case FFK_INT64: return cast_out<int64_t>(who, st, out_dtype, in, out, n, backward);
    case FFK_HALF: return cast_out<_Float16>(who, st, out_dtype, in, out, n, backward);
    case FFK_FLOAT: return cast_out<float>(who, st, out_dtype, in, out, n, backward);
    case FFK_DOUBLE: return cast_out<double>(who, st, out_dtype, in, out, n, backward);
    case FFK_BF16: return cast_out<bf16>(who, st, out_dtype, in, out, n, backward);
    default: return fail(FFK_ERR_UNSUPPORTED, "%s: input dtype %d not supported", who, in_dtype);
  }
}

}  // namespace ffk

using namespace ffk;

extern "C" int ffk_cast_forward(ffk_stream_t stream, int input_dtype, int output_dtype,
                                void const *input, void *output, int64_t num_elements) {
  return cast_any("cast_forward", stream, input_dtype, output_dtype, input, output, num_elements, false);
}

extern "C" int ffk_cast_backward(ffk_stream_t stream, int output_grad_dtype,
                                 int input_grad_dtype, void const *output_grad,
                                 void *input_grad, int64_t num_elements) {
  return cast_any("cast_backward", stream, output_grad_dtype, input_grad_dtype, output_grad,
                  input_grad, num_elements, true);
}
