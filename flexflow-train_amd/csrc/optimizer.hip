// SGD and Adam parameter updates for gfx950 (reference: sgd_update / adam_update
// and their *_update_task launchers, lib/kernels/src/cuda/optimizer_kernels.cu:
// 23-133; CPU SGD lib/kernels/src/kernels/optimizer_kernels_cpu.cc:10-60).
//
// One pass, 16 bytes per lane per access, every operand read once.  Each
// arithmetic step is a separately rounded fp32 operation (no fused
// multiply-add), so the result equals the reference's CPU evaluation, which
// composes rounded tensor ops, bit for bit.  Weights and optimizer state are
// fp32 as in the reference; the gradient may be fp32 or bf16, replicas of the
// gradient ([num_replicas][n]) are summed in replica order like the
// parameter-server launcher does, and an optional bf16 copy of the updated
// weights can be written in the same pass (for bf16 compute kernels).
#include "ffk_common.h"

namespace ffk {

constexpr int kOptThreads = 256;
constexpr int kOptUnroll = 2;  // Adam: vectors per thread

// 16-byte accesses; STREAM: past the caches (parameter sets larger than the last-level cache
// are touched once per step and never found there again)
template <bool STREAM, typename VT>
__device__ __forceinline__ VT opt_load(VT const *p) {
  if constexpr (STREAM) return __builtin_nontemporal_load(p);
  else return *p;
}
template <bool STREAM, typename VT>
__device__ __forceinline__ void opt_store(VT *p, VT v) {
  if constexpr (STREAM) __builtin_nontemporal_store(v, p);
  else *p = v;
}

template <bool STREAM>
__device__ __forceinline__ void load_grad_sum(float const *g, int64_t i, int64_t n,
                                              int replicas, float (&v)[4]) {
  f32x4 r = opt_load<STREAM>(reinterpret_cast<f32x4 const *>(g + i));
  v[0] = r[0]; v[1] = r[1]; v[2] = r[2]; v[3] = r[3];
  for (int k = 1; k < replicas; k++) {
    f32x4 x = opt_load<STREAM>(reinterpret_cast<f32x4 const *>(g + (int64_t)k * n + i));
#pragma unroll
    for (int e = 0; e < 4; e++) v[e] = __fadd_rn(v[e], x[e]);
  }
}

template <bool STREAM>
__device__ __forceinline__ void load_grad_sum(bf16 const *g, int64_t i, int64_t n,
                                              int replicas, float (&v)[4]) {
  u32x2 r = opt_load<STREAM>(reinterpret_cast<u32x2 const *>(g + i));
  v[0] = __uint_as_float(r[0] << 16);
  v[1] = __uint_as_float(r[0] & 0xffff0000u);
  v[2] = __uint_as_float(r[1] << 16);
  v[3] = __uint_as_float(r[1] & 0xffff0000u);
  for (int k = 1; k < replicas; k++) {
    u32x2 x = opt_load<STREAM>(reinterpret_cast<u32x2 const *>(g + (int64_t)k * n + i));
    v[0] = __fadd_rn(v[0], __uint_as_float(x[0] << 16));
    v[1] = __fadd_rn(v[1], __uint_as_float(x[0] & 0xffff0000u));
    v[2] = __fadd_rn(v[2], __uint_as_float(x[1] << 16));
    v[3] = __fadd_rn(v[3], __uint_as_float(x[1] & 0xffff0000u));
  }
}

template <typename GT>
__device__ __forceinline__ float load_grad_sum1(GT const *g, int64_t i, int64_t n, int replicas) {
  float v = VecIO<GT>::load1(g + i);
  for (int k = 1; k < replicas; k++) v = __fadd_rn(v, VecIO<GT>::load1(g + (int64_t)k * n + i));
  return v;
}

struct SgdParams {
  float lr, weight_decay, momentum;
  int nesterov;
};

__device__ __forceinline__ float sgd_step(float g, float &w, float *v, SgdParams const &p) {
  // gt = g + wd * w ; V = V * momentum + gt ; gt = nesterov ? gt + momentum * V : V ; W -= lr * gt
  float gt = __fadd_rn(g, __fmul_rn(p.weight_decay, w));
  if (p.momentum > 0.0f) {
    float vn = __fadd_rn(__fmul_rn(*v, p.momentum), gt);
    *v = vn;
    gt = p.nesterov ? __fadd_rn(gt, __fmul_rn(p.momentum, vn)) : vn;
  }
  w = __fsub_rn(w, __fmul_rn(p.lr, gt));
  return w;
}

template <typename GT, bool STREAM>
__global__ __launch_bounds__(kOptThreads) void sgd_update_kernel(
    GT const *__restrict__ grad, float *W, float *V, bf16 *W_lowp, int64_t n,
    int replicas, SgdParams p) {
  int64_t const q = (int64_t)blockIdx.x * kOptThreads + threadIdx.x;
  int64_t const i = q * 4;
  if (i + 4 <= n) {
    float g[4];
    load_grad_sum<STREAM>(grad, i, n, replicas, g);
    f32x4 w = opt_load<STREAM>(reinterpret_cast<f32x4 const *>(W + i));
    f32x4 v = {0.0f, 0.0f, 0.0f, 0.0f};
    if (p.momentum > 0.0f) v = opt_load<STREAM>(reinterpret_cast<f32x4 const *>(V + i));
    float wv[4] = {w[0], w[1], w[2], w[3]}, vv[4] = {v[0], v[1], v[2], v[3]};
#pragma unroll
    for (int e = 0; e < 4; e++) sgd_step(g[e], wv[e], &vv[e], p);
    opt_store<STREAM>(reinterpret_cast<f32x4 *>(W + i), f32x4{wv[0], wv[1], wv[2], wv[3]});
    if (p.momentum > 0.0f) opt_store<STREAM>(reinterpret_cast<f32x4 *>(V + i), f32x4{vv[0], vv[1], vv[2], vv[3]});
    if (W_lowp != nullptr) {
      u32x2 lo = {pack_bf16x2(wv[0], wv[1]), pack_bf16x2(wv[2], wv[3])};
      opt_store<STREAM>(reinterpret_cast<u32x2 *>(W_lowp + i), lo);
    }
  } else {
    for (int64_t j = i; j < n; j++) {
      float g = load_grad_sum1<GT>(grad, j, n, replicas);
      float w = W[j], v = p.momentum > 0.0f ? V[j] : 0.0f;
      sgd_step(g, w, &v, p);
      W[j] = w;
      if (p.momentum > 0.0f) V[j] = v;
      if (W_lowp != nullptr) VecIO<bf16>::store1(W_lowp + j, w);
    }
  }
}

struct AdamParams {
  float alpha_t, beta1, beta2, weight_decay, epsilon;
};

__device__ __forceinline__ void adam_step(float g, float &w, float &m, float &v, AdamParams const &p) {
  // gt = g + wd * W ; mt = b1 * M + (1 - b1) * gt ; vt = b2 * V + (1 - b2) * gt * gt
  // W -= alpha_t * mt / (sqrt(vt) + eps)          (optimizer_kernels.cu:111-133)
  float gt = __fadd_rn(g, __fmul_rn(p.weight_decay, w));
  float mt = __fadd_rn(__fmul_rn(p.beta1, m), __fmul_rn(__fsub_rn(1.0f, p.beta1), gt));
  float vt = __fadd_rn(__fmul_rn(p.beta2, v), __fmul_rn(__fmul_rn(__fsub_rn(1.0f, p.beta2), gt), gt));
  m = mt;
  v = vt;
  // plain sqrtf and / are the correctly rounded ones (hipcc's default
  // -fhip-fp32-correctly-rounded-divide-sqrt); this file is built without
  // contraction, so the expression below rounds step by step
  float const den = sqrtf(vt) + p.epsilon;
  float const num = p.alpha_t * mt;
  float const q = num / den;
  w = w - q;
}

template <typename GT, bool STREAM>
__global__ __launch_bounds__(kOptThreads) void adam_update_kernel(
    GT const *__restrict__ grad, float *W, float *M, float *V, bf16 *W_lowp,
    int64_t n, int replicas, AdamParams p) {
  // kOptUnroll vectors of 4 parameters per thread, a workgroup's vectors interleaved: all loads
  // of a thread are issued before the first arithmetic, which keeps more bytes in flight
  int64_t const first = ((int64_t)blockIdx.x * kOptThreads * kOptUnroll + threadIdx.x) * 4;
  if (first + (int64_t)(kOptUnroll - 1) * kOptThreads * 4 + 4 <= n) {
    float g[kOptUnroll][4];
    f32x4 w[kOptUnroll], m[kOptUnroll], v[kOptUnroll];
#pragma unroll
    for (int u = 0; u < kOptUnroll; u++) {
      int64_t const i = first + (int64_t)u * kOptThreads * 4;
      load_grad_sum<STREAM>(grad, i, n, replicas, g[u]);
      w[u] = opt_load<STREAM>(reinterpret_cast<f32x4 const *>(W + i));
      m[u] = opt_load<STREAM>(reinterpret_cast<f32x4 const *>(M + i));
      v[u] = opt_load<STREAM>(reinterpret_cast<f32x4 const *>(V + i));
    }
#pragma unroll
    for (int u = 0; u < kOptUnroll; u++) {
      int64_t const i = first + (int64_t)u * kOptThreads * 4;
      float wv[4] = {w[u][0], w[u][1], w[u][2], w[u][3]}, mv[4] = {m[u][0], m[u][1], m[u][2], m[u][3]},
            vv[4] = {v[u][0], v[u][1], v[u][2], v[u][3]};
#pragma unroll
      for (int e = 0; e < 4; e++) adam_step(g[u][e], wv[e], mv[e], vv[e], p);
      opt_store<STREAM>(reinterpret_cast<f32x4 *>(W + i), f32x4{wv[0], wv[1], wv[2], wv[3]});
      opt_store<STREAM>(reinterpret_cast<f32x4 *>(M + i), f32x4{mv[0], mv[1], mv[2], mv[3]});
      opt_store<STREAM>(reinterpret_cast<f32x4 *>(V + i), f32x4{vv[0], vv[1], vv[2], vv[3]});
      if (W_lowp != nullptr) {
        u32x2 lo = {pack_bf16x2(wv[0], wv[1]), pack_bf16x2(wv[2], wv[3])};
        opt_store<STREAM>(reinterpret_cast<u32x2 *>(W_lowp + i), lo);
      }
    }
  } else {
    // the last workgroup: element by element
    for (int u = 0; u < kOptUnroll; u++) {
      int64_t const i = first + (int64_t)u * kOptThreads * 4;
      for (int64_t j = i; j < min(i + 4, n); j++) {
        float g = load_grad_sum1<GT>(grad, j, n, replicas);
        float w = W[j], m = M[j], v = V[j];
        adam_step(g, w, m, v, p);
        W[j] = w;
        M[j] = m;
        V[j] = v;
        if (W_lowp != nullptr) VecIO<bf16>::store1(W_lowp + j, w);
      }
    }
  }
}

static int check_update(char const *who, int grad_dtype, void const *grad, int64_t n,
                        int replicas, void const *w, void const *lowp) {
  FFK_REQUIRE(grad_dtype == FFK_FLOAT || grad_dtype == FFK_BF16,
              "%s: gradient dtype %d not supported (float or bf16)", who, grad_dtype);
  FFK_REQUIRE(n >= 0 && replicas >= 1, "%s: bad size", who);
  if (n == 0) return FFK_OK;
  FFK_REQUIRE(grad && w, "%s: NULL tensor", who);
  // replica r of the gradient starts at element r * n: vector access needs that aligned
  FFK_REQUIRE(aligned16(grad) && aligned16(w) && (lowp == nullptr || aligned16(lowp)) &&
                  (replicas == 1 || n % 8 == 0),
              "%s: tensors must be 16-byte aligned (and n a multiple of 8 with replicas)", who);
  return FFK_OK;
}

}  // namespace ffk

using namespace ffk;

extern "C" int ffk_sgd_update(ffk_stream_t stream, int grad_dtype, float lr,
                              float momentum, int nesterov, float weight_decay,
                              void const *weight_grad, int64_t num_elements,
                              int num_replicas, float *weight, float *sgd_v,
                              void *weight_lowp) {
  int rc = check_update("sgd_update", grad_dtype, weight_grad, num_elements, num_replicas, weight, weight_lowp);
  if (rc != FFK_OK) return rc;
  if (num_elements == 0) return FFK_OK;
  // the reference asserts sgd_v.has_value() == (momentum > 0) (optimizer_kernels.cc:18)
  FFK_REQUIRE((sgd_v != nullptr) == (momentum > 0.0f),
              "sgd_update: sgd_v must be given exactly when momentum > 0");
  FFK_REQUIRE(sgd_v == nullptr || aligned16(sgd_v), "sgd_update: sgd_v must be 16-byte aligned");
  SgdParams p{lr, weight_decay, momentum, nesterov != 0};
  unsigned const blocks = (unsigned)ceil_div(ceil_div(num_elements, 4), kOptThreads);
  hipStream_t st = as_stream(stream);
  // weights, velocity and gradient together: what one step walks through
  bool const past_caches = stream_past_caches(num_elements, 12);
#define FFK_SGD(GT_, S_)                                                       \
  sgd_update_kernel<GT_, S_><<<blocks, kOptThreads, 0, st>>>(                  \
      static_cast<GT_ const *>(weight_grad), weight, sgd_v, static_cast<bf16 *>(weight_lowp), \
      num_elements, num_replicas, p)
  if (grad_dtype == FFK_FLOAT) {
    if (past_caches) FFK_SGD(float, true); else FFK_SGD(float, false);
  } else {
    if (past_caches) FFK_SGD(bf16, true); else FFK_SGD(bf16, false);
  }
#undef FFK_SGD
  FFK_CHECK_LAUNCH();
  return FFK_OK;
}

extern "C" int ffk_adam_update(ffk_stream_t stream, int grad_dtype, float alpha_t,
                               float beta1, float beta2, float weight_decay,
                               float epsilon, void const *weight_grad,
                               int64_t num_elements, int num_replicas,
                               float *weight, float *adam_v, float *adam_m,
                               void *weight_lowp) {
  int rc = check_update("adam_update", grad_dtype, weight_grad, num_elements, num_replicas, weight, weight_lowp);
  if (rc != FFK_OK) return rc;
  if (num_elements == 0) return FFK_OK;
  FFK_REQUIRE(adam_v && adam_m && aligned16(adam_v) && aligned16(adam_m),
              "adam_update: adam_v / adam_m must be given and 16-byte aligned");
  AdamParams p{alpha_t, beta1, beta2, weight_decay, epsilon};
  unsigned const blocks = (unsigned)ceil_div(ceil_div(num_elements, 4), kOptThreads * kOptUnroll);
  hipStream_t st = as_stream(stream);
  bool const past_caches = stream_past_caches(num_elements, 16);
#define FFK_ADAM(GT_, S_)                                                      \
  adam_update_kernel<GT_, S_><<<blocks, kOptThreads, 0, st>>>(                 \
      static_cast<GT_ const *>(weight_grad), weight, adam_m, adam_v, static_cast<bf16 *>(weight_lowp), \
      num_elements, num_replicas, p)
  if (grad_dtype == FFK_FLOAT) {
    if (past_caches) FFK_ADAM(float, true); else FFK_ADAM(float, false);
  } else {
    if (past_caches) FFK_ADAM(bf16, true); else FFK_ADAM(bf16, false);
  }
#undef FFK_ADAM
  FFK_CHECK_LAUNCH();
  return FFK_OK;
}
