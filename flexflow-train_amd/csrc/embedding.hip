// Embedding gather (forward) and scatter-add (backward) for gfx950.
//
// forward : output[b,:] = sum_j weight[indices[b,j],:], 16 bytes per lane per
//           row access, the index of a bag entry read once per lane group and
//           int64 offsets throughout (the reference does one element per
//           thread with `int` offsets and re-reads the index per element,
//           lib/kernels/src/cuda/embedding_kernels.cu:48-125).
// backward: weight_grad[indices[b,j],:] += output_grad[b,:] with hardware fp32
//           atomics, one wave instruction covering 64 consecutive floats of a
//           row (reference: atomicAdd per element, embedding_kernels.cu:128-317).
// Indices outside [0, num_entries) are skipped (the reference reads or writes
// out of bounds for them).
#include "ffk_common.h"

namespace ffk {

constexpr int kEmbThreads = 256;

template <typename OT, int V>
__device__ __forceinline__ void store_out(OT *p, float const (&v)[V]);

template <>
__device__ __forceinline__ void store_out<float, 4>(float *p, float const (&v)[4]) {
  *reinterpret_cast<f32x4 *>(p) = f32x4{v[0], v[1], v[2], v[3]};
}
template <>
__device__ __forceinline__ void store_out<float, 8>(float *p, float const (&v)[8]) {
  *reinterpret_cast<f32x4 *>(p) = f32x4{v[0], v[1], v[2], v[3]};
  *reinterpret_cast<f32x4 *>(p + 4) = f32x4{v[4], v[5], v[6], v[7]};
}
template <>
__device__ __forceinline__ void store_out<bf16, 4>(bf16 *p, float const (&v)[4]) {
  *reinterpret_cast<u32x2 *>(p) = u32x2{pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
}
template <>
__device__ __forceinline__ void store_out<bf16, 8>(bf16 *p, float const (&v)[8]) {
  VecIO<bf16>::store(p, v);
}

// One thread per (bag, 16-byte vector of the row).
template <typename IT, typename WT, typename OT>
__global__ __launch_bounds__(kEmbThreads) void embedding_fwd_vec_kernel(
    IT const *__restrict__ idx, OT *__restrict__ out, WT const *__restrict__ W,
    int64_t num_bags, int bag, int nvec, int64_t dim, int64_t num_entries,
    float scale) {
  constexpr int V = VecIO<WT>::kVec;
  int64_t const total = num_bags * nvec;
  int64_t const stride = (int64_t)gridDim.x * kEmbThreads;
  for (int64_t i = (int64_t)blockIdx.x * kEmbThreads + threadIdx.x; i < total; i += stride) {
    int64_t const b = i / nvec;
    int const v = (int)(i % nvec);
    float acc[V];
#pragma unroll
    for (int e = 0; e < V; e++) acc[e] = 0.0f;
    IT const *ib = idx + b * bag;
    int j = 0;
    for (; j + 4 <= bag; j += 4) {  // four row reads in flight
      int64_t r[4];
      float w[4][V];
#pragma unroll
      for (int u = 0; u < 4; u++) r[u] = (int64_t)ib[j + u];
#pragma unroll
      for (int u = 0; u < 4; u++) {
        bool ok = (uint64_t)r[u] < (uint64_t)num_entries;
        VecIO<WT>::load(W + (ok ? r[u] : 0) * dim + (int64_t)v * V, w[u]);
        if (!ok) {
#pragma unroll
          for (int e = 0; e < V; e++) w[u][e] = 0.0f;
        }
      }
#pragma unroll
      for (int u = 0; u < 4; u++)
#pragma unroll
        for (int e = 0; e < V; e++) acc[e] = acc[e] + w[u][e];
    }
    for (; j < bag; j++) {
      int64_t r = (int64_t)ib[j];
      if ((uint64_t)r < (uint64_t)num_entries) {
        float w[V];
        VecIO<WT>::load(W + r * dim + (int64_t)v * V, w);
#pragma unroll
        for (int e = 0; e < V; e++) acc[e] = acc[e] + w[e];
      }
    }
    if (scale != 1.0f) {
#pragma unroll
      for (int e = 0; e < V; e++) acc[e] *= scale;
    }
    store_out<OT, V>(out + b * dim + (int64_t)v * V, acc);
  }
}

template <typename IT, typename WT, typename OT>
__global__ __launch_bounds__(kEmbThreads) void embedding_fwd_scalar_kernel(
    IT const *__restrict__ idx, OT *__restrict__ out, WT const *__restrict__ W,
    int64_t num_bags, int bag, int64_t dim, int64_t num_entries, float scale) {
  int64_t const total = num_bags * dim;
  int64_t const stride = (int64_t)gridDim.x * kEmbThreads;
  for (int64_t i = (int64_t)blockIdx.x * kEmbThreads + threadIdx.x; i < total; i += stride) {
    int64_t const b = i / dim, d = i % dim;
    float acc = 0.0f;
    for (int j = 0; j < bag; j++) {
      int64_t r = (int64_t)idx[b * bag + j];
      if ((uint64_t)r < (uint64_t)num_entries) {
        acc = acc + VecIO<WT>::load1(W + r * dim + d);
      }
    }
    if (scale != 1.0f) acc *= scale;
    VecIO<OT>::store1(out + b * dim + d, acc);
  }
}

// One wave per (bag, 64-float column segment): every atomic instruction of the
// wave covers 256 contiguous bytes of one weight-gradient row.
template <typename IT, typename GT>
__global__ __launch_bounds__(kEmbThreads) void embedding_bwd_atomic_kernel(
    IT const *__restrict__ idx, GT const *__restrict__ dY, float *dW,
    int64_t num_bags, int bag, int64_t dim, int64_t num_entries, float scale) {
  int const lane = threadIdx.x & 63;
  int64_t const segs = ceil_div(dim, 64);
  int64_t const total = num_bags * segs;
  int64_t const wave0 = ((int64_t)blockIdx.x * kEmbThreads + threadIdx.x) >> 6;
  int64_t const nwaves = ((int64_t)gridDim.x * kEmbThreads) >> 6;
  for (int64_t w = wave0; w < total; w += nwaves) {
    int64_t const b = w / segs;
    int64_t const d = (w % segs) * 64 + lane;
    if (d < dim) {
      float g = VecIO<GT>::load1(dY + b * dim + d);
      if (scale != 1.0f) g *= scale;
      for (int j = 0; j < bag; j++) {
        int64_t r = (int64_t)idx[b * bag + j];
        if ((uint64_t)r < (uint64_t)num_entries) {
          atomicAdd(dW + r * dim + d, g);
        }
      }
    }
  }
}

static int emb_grid(int64_t threads_needed) {
  int64_t b = ceil_div(threads_needed > 0 ? threads_needed : 1, kEmbThreads);
  int64_t const cap = (int64_t)kNumCU * 32;
  return (int)(b < cap ? b : cap);
}

template <typename IT, typename WT, typename OT>
static int emb_forward(hipStream_t st, void const *indices, void *output,
                       void const *weight, int64_t num_bags, int64_t bag,
                       int64_t dim, int64_t num_entries, float scale) {
  constexpr int V = VecIO<WT>::kVec;
  IT const *I = static_cast<IT const *>(indices);
  WT const *W = static_cast<WT const *>(weight);
  OT *O = static_cast<OT *>(output);
  if (dim % V == 0 && aligned16(weight) && aligned16(output)) {
    int nvec = (int)(dim / V);
    embedding_fwd_vec_kernel<IT, WT, OT><<<emb_grid(num_bags * nvec), kEmbThreads, 0, st>>>(
        I, O, W, num_bags, (int)bag, nvec, dim, num_entries, scale);
  } else {
    embedding_fwd_scalar_kernel<IT, WT, OT><<<emb_grid(num_bags * dim), kEmbThreads, 0, st>>>(
        I, O, W, num_bags, (int)bag, dim, num_entries, scale);
  }
  FFK_CHECK_LAUNCH();
  return FFK_OK;
}

template <typename IT, typename GT>
static int emb_backward(hipStream_t st, void const *indices, void const *dy,
                        float *dw, int64_t num_bags, int64_t bag, int64_t dim,
                        int64_t num_entries, float scale) {
  int64_t waves = num_bags * ceil_div(dim, 64);
  embedding_bwd_atomic_kernel<IT, GT><<<emb_grid(waves * 64), kEmbThreads, 0, st>>>(
      static_cast<IT const *>(indices), static_cast<GT const *>(dy), dw, num_bags,
      (int)bag, dim, num_entries, scale);
  FFK_CHECK_LAUNCH();
  return FFK_OK;
}

static int check_common(char const *who, int aggr, int64_t num_bags, int64_t bag,
                        int64_t dim, int64_t num_entries) {
  FFK_REQUIRE(num_bags >= 0 && bag > 0 && dim > 0 && num_entries > 0, "%s: bad shape", who);
  FFK_REQUIRE(bag < (1ll << 31), "%s: bag too large", who);
  FFK_REQUIRE(aggr >= FFK_AGGR_NONE && aggr <= FFK_AGGR_AVG, "%s: bad aggregate op %d", who, aggr);
  FFK_REQUIRE(aggr != FFK_AGGR_NONE || bag == 1, "%s: bag must be 1 without an aggregate op", who);
  return FFK_OK;
}

}  // namespace ffk

using namespace ffk;

extern "C" int ffk_embedding_forward(ffk_stream_t stream, int index_dtype,
                                     int weight_dtype, int output_dtype,
                                     void const *indices, void *output,
                                     void const *weight, int aggr,
                                     int64_t num_bags, int64_t bag, int64_t dim,
                                     int64_t num_entries) {
  int rc = check_common("embedding_forward", aggr, num_bags, bag, dim, num_entries);
  if (rc != FFK_OK) return rc;
  if (num_bags == 0) return FFK_OK;
  FFK_REQUIRE(indices && output && weight, "embedding_forward: NULL tensor");
  float scale = aggr == FFK_AGGR_AVG ? 1.0f / (float)bag : 1.0f;
  hipStream_t st = as_stream(stream);
#define FFK_EMB_FWD(IT, WT, OT)                                                \
  return emb_forward<IT, WT, OT>(st, indices, output, weight, num_bags, bag, dim, num_entries, scale)
  if (index_dtype == FFK_INT32) {
    if (weight_dtype == FFK_FLOAT && output_dtype == FFK_FLOAT) FFK_EMB_FWD(int32_t, float, float);
    if (weight_dtype == FFK_FLOAT && output_dtype == FFK_BF16) FFK_EMB_FWD(int32_t, float, bf16);
    if (weight_dtype == FFK_BF16 && output_dtype == FFK_BF16) FFK_EMB_FWD(int32_t, bf16, bf16);
    if (weight_dtype == FFK_BF16 && output_dtype == FFK_FLOAT) FFK_EMB_FWD(int32_t, bf16, float);
  } else if (index_dtype == FFK_INT64) {
    if (weight_dtype == FFK_FLOAT && output_dtype == FFK_FLOAT) FFK_EMB_FWD(int64_t, float, float);
    if (weight_dtype == FFK_FLOAT && output_dtype == FFK_BF16) FFK_EMB_FWD(int64_t, float, bf16);
    if (weight_dtype == FFK_BF16 && output_dtype == FFK_BF16) FFK_EMB_FWD(int64_t, bf16, bf16);
    if (weight_dtype == FFK_BF16 && output_dtype == FFK_FLOAT) FFK_EMB_FWD(int64_t, bf16, float);
  }
#undef FFK_EMB_FWD
  return fail(FFK_ERR_UNSUPPORTED,
              "embedding_forward: dtypes (index %d, weight %d, output %d) not supported",
              index_dtype, weight_dtype, output_dtype);
}

extern "C" size_t ffk_embedding_backward_workspace_bytes(int64_t num_indices,
                                                         int64_t num_entries) {
  (void)num_entries;
  // keys + positions, double-buffered, plus per-pass digit histograms
  return (size_t)num_indices * 16 + ((size_t)1 << 20);
}

extern "C" int ffk_embedding_backward(ffk_stream_t stream, int index_dtype,
                                      int output_grad_dtype,
                                      void const *indices,
                                      void const *output_grad,
                                      float *weight_grad, int aggr,
                                      int64_t num_bags, int64_t bag,
                                      int64_t dim, int64_t num_entries,
                                      int deterministic, void *workspace,
                                      size_t workspace_bytes) {
  int rc = check_common("embedding_backward", aggr, num_bags, bag, dim, num_entries);
  if (rc != FFK_OK) return rc;
  if (num_bags == 0) return FFK_OK;
  FFK_REQUIRE(indices && output_grad && weight_grad, "embedding_backward: NULL tensor");
  (void)workspace;
  (void)workspace_bytes;
  if (deterministic) {
    return fail(FFK_ERR_UNSUPPORTED, "embedding_backward: deterministic mode not built yet");
  }
  float scale = aggr == FFK_AGGR_AVG ? 1.0f / (float)bag : 1.0f;
  hipStream_t st = as_stream(stream);
#define FFK_EMB_BWD(IT, GT)                                                    \
  return emb_backward<IT, GT>(st, indices, output_grad, weight_grad, num_bags, bag, dim, num_entries, scale)
  if (index_dtype == FFK_INT32) {
    if (output_grad_dtype == FFK_FLOAT) FFK_EMB_BWD(int32_t, float);
    if (output_grad_dtype == FFK_BF16) FFK_EMB_BWD(int32_t, bf16);
  } else if (index_dtype == FFK_INT64) {
    if (output_grad_dtype == FFK_FLOAT) FFK_EMB_BWD(int64_t, float);
    if (output_grad_dtype == FFK_BF16) FFK_EMB_BWD(int64_t, bf16);
  }
#undef FFK_EMB_BWD
  return fail(FFK_ERR_UNSUPPORTED,
              "embedding_backward: dtypes (index %d, grad %d) not supported",
              index_dtype, output_grad_dtype);
}
