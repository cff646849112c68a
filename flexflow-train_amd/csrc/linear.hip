// Linear forward/backward for gfx950.
//
// forward : output = act(input . weight^T + bias), bias and activation fused
//           into the GEMM epilogue (the reference runs a second rank-1 GEMM for
//           the bias, lib/kernels/src/cuda/ops/linear_kernels.cu:163, and never
//           applies the activation on the GPU, :183-200; its CPU path does,
//           lib/kernels/src/kernels/linear_kernels_cpu.cc:33-42).
// backward: g = act'(.) * output_grad into the caller's workspace (the
//           reference cudaMallocs a copy of output_grad per call,
//           lib/kernels/src/kernels/linear_kernels.cc:104-106), then three
//           products: input_grad (+)= g . W, weight_grad (+)= g^T . X,
//           bias_grad (+)= column sums of g (linear_kernels.cu:249-334).
#include "elementwise.h"
#include "gemm.h"

namespace ffk {

// in = (output, output_grad); out = g
template <int ACT, int MODE>
struct ActGrad {
  __device__ __forceinline__ void operator()(float const (&in)[2],
                                             float (&out)[1]) const {
    float y = in[0], dy = in[1];
    float g;
    if (ACT == FFK_ACT_RELU) {
      if (MODE == 1) {
        g = dy > 0.0f ? 1.0f : 0.0f;  // linear_kernels_cpu.cc:46-52,69-71
      } else {
        g = y > 0.0f ? dy : 0.0f;     // cuda_helper.cu:60-64
      }
    } else if (ACT == FFK_ACT_SIGMOID) {
      g = dy * y * (1.0f - y);        // cuda_helper.cu:87-91
    } else {
      g = dy * (1.0f - y * y);        // tanh
    }
    out[0] = g;
  }
};

template <typename T>
static hipError_t act_grad(hipStream_t st, int act, int mode, void const *y,
                           void const *dy, void *g, int64_t n) {
  EwArgs<T, 2, 1> a;
  a.in[0] = static_cast<T const *>(y);
  a.in[1] = static_cast<T const *>(dy);
  a.in_elems[0] = n;
  a.in_elems[1] = n;
  a.out[0] = static_cast<T *>(g);
  a.n = n;
  if (act == FFK_ACT_RELU && mode == 1) return ew_launch<T, 2, 1>(st, a, ActGrad<FFK_ACT_RELU, 1>{});
  if (act == FFK_ACT_RELU) return ew_launch<T, 2, 1>(st, a, ActGrad<FFK_ACT_RELU, 0>{});
  if (act == FFK_ACT_SIGMOID) return ew_launch<T, 2, 1>(st, a, ActGrad<FFK_ACT_SIGMOID, 0>{});
  return ew_launch<T, 2, 1>(st, a, ActGrad<FFK_ACT_TANH, 0>{});
}

static size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

// in = (weight, weight_grad); out = weight_grad + lambda * weight
struct L2RegGrad {
  float lambda;
  __device__ __forceinline__ void operator()(float const (&in)[2], float (&out)[1]) const {
    out[0] = in[1] + lambda * in[0];
  }
};

template <typename T>
static hipError_t l2_reg_grad(hipStream_t st, void const *w, void *dw, int64_t n, float lambda) {
  EwArgs<T, 2, 1> a;
  a.in[0] = static_cast<T const *>(w);
  a.in[1] = static_cast<T const *>(dw);
  a.in_elems[0] = n;
  a.in_elems[1] = n;
  a.out[0] = static_cast<T *>(dw);
  a.n = n;
  return ew_launch<T, 2, 1>(st, a, L2RegGrad{lambda});
}

// ---------------------------------------------------------------------------
// The whole backward of a small fp32 Linear in ONE launch.  At sizes like the
// reference's CPU-runnable case ([32,64] . [128,64]^T) every kernel is a few
// microseconds of launch latency around almost no work, so the activation
// gradient, the two products and the bias sums, which are independent given
// (output, output_grad), run as jobs of one grid: workgroups [0, tiles_dx)
// compute 64x64 tiles of input_grad, the next tiles_dw ones tiles of
// weight_grad, the rest 64 columns of bias_grad each.  g = act'(output) *
// output_grad is applied where an operand element is loaded, never stored.
// ---------------------------------------------------------------------------
struct SmallLinearBwd {
  float const *y, *dy, *x, *w;
  float *dx, *dw, *db;
  int batch, in_dim, out_dim;
  int act, relu_mode, accumulate;  // accumulate: FFK_ACC_* bits
  int tiles_dx, tiles_dw;
};

// ACT is a template argument of the kernel: a run-time switch here puts a branch and a wait
// between every two loads of a thread, and the kernel's time is its round trips to memory.
template <int ACT>
__device__ __forceinline__ float small_act_grad(int mode, float y, float dy) {
  if constexpr (ACT == FFK_ACT_RELU) {
    return mode == 1 ? (dy > 0.0f ? 1.0f : 0.0f) : (y > 0.0f ? dy : 0.0f);
  } else if constexpr (ACT == FFK_ACT_SIGMOID) {
    return dy * y * (1.0f - y);
  } else if constexpr (ACT == FFK_ACT_TANH) {
    return dy * (1.0f - y * y);
  } else {
    return dy;
  }
}

// One 64x64 tile of sum_k a(m, k) * b(k, n), handed element by element to store(m, n, value).  a
// and b clamp their coordinates into the problem and return what lies there: rows and columns
// past the edge give values that are never stored, k past the edge is zeroed here when the tile
// is written to LDS (a select on a loaded value any earlier is a wait for that load).  A_KFAST: consecutive lanes walk k of the A operand (it
// lies [M][K]); otherwise m; B_KFAST likewise for B lying [N][K].  A k-tile is 64 deep, all of a thread's 32 loads are issued
// before the first is waited for, and the next k-tile's are issued before this one is multiplied: at these sizes the
// time is the number of round trips to memory, not the arithmetic.
constexpr int kSmallBK = 64;
constexpr int kSmallMaxDepth = 1024;  // longest reduction the one-launch kernels take (16 k-tiles)
// a returns what it loaded (a float, or the pair an activation gradient is made of) and av turns
// that into the operand's value when the tile is written to LDS, one k-tile later: arithmetic on a
// loaded value any earlier would make the wave wait for the load it is meant to run under.
template <bool A_KFAST, bool B_KFAST, typename FA, typename FAV, typename FB, typename FS>
__device__ __forceinline__ void small_f32_tile(FA a, FAV av, FB b, int M, int N, int K, int m0, int n0, FS store,
                                               float (&As)[kSmallBK][68], float (&Bs)[kSmallBK][68],
                                               float const *prior = nullptr, int64_t prior_ld = 0) {
  int const t = threadIdx.x, lane = t & 63, wave = t >> 6;
  int const wm0 = (wave >> 1) * 32, wn0 = (wave & 1) * 32;
  f32x16 acc;
#pragma unroll
  for (int r = 0; r < 16; r++) acc[r] = 0.0f;
  decltype(a(0, 0)) ra[16];
  float rb[16];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int i = 0; i < 16; i++) {
      int const k = A_KFAST ? (t & 63) : (t >> 6) + 4 * i;
      int const m = A_KFAST ? (t >> 6) + 4 * i : (t & 63);
      int const kb = B_KFAST ? (t & 63) : (t >> 6) + 4 * i;
      int const n = B_KFAST ? (t >> 6) + 4 * i : (t & 63);
      ra[i] = a(m0 + m, k0 + k);
      rb[i] = b(k0 + kb, n0 + n);
    }
  };
  fetch(0);
  for (int k0 = 0; k0 < K; k0 += kSmallBK) {
#pragma unroll
    for (int i = 0; i < 16; i++) {
      int const k = A_KFAST ? (t & 63) : (t >> 6) + 4 * i;
      int const m = A_KFAST ? (t >> 6) + 4 * i : (t & 63);
      int const kb = B_KFAST ? (t & 63) : (t >> 6) + 4 * i;
      int const n = B_KFAST ? (t >> 6) + 4 * i : (t & 63);
      As[k][m] = k0 + k < K ? av(ra[i]) : 0.0f;
      Bs[kb][n] = k0 + kb < K ? rb[i] : 0.0f;
    }
    __syncthreads();
    if (k0 + kSmallBK < K) fetch(k0 + kSmallBK);  // on its way while this tile is multiplied
#pragma unroll
    for (int kk = 0; kk < kSmallBK / 2; kk++) {
      float const av = As[2 * kk + (lane >> 5)][wm0 + (lane & 31)];
      float const bv = Bs[2 * kk + (lane >> 5)][wn0 + (lane & 31)];
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv, acc, 0, 0, 0);
    }
    __syncthreads();
  }
  int const n = n0 + wn0 + (lane & 31);
  if (n < N) {
    if (prior != nullptr) {  // accumulating: what the destination holds, all 16 loads in flight together
      float old[16];
#pragma unroll
      for (int r = 0; r < 16; r++) {
        int const m = m0 + wm0 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        old[r] = prior[(int64_t)(m < M ? m : M - 1) * prior_ld + n];
      }
#pragma unroll
      for (int r = 0; r < 16; r++) acc[r] = old[r] + acc[r];
    }
#pragma unroll
    for (int r = 0; r < 16; r++) {
      int const m = m0 + wm0 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
      if (m < M) store(m, n, acc[r]);
    }
  }
}

template <int ACT>
__global__ __launch_bounds__(256) void linear_small_bwd_f32_kernel(SmallLinearBwd p) {
  __shared__ float As[kSmallBK][68], Bs[kSmallBK][68];
  int const bid = blockIdx.x;
  // g[batch, out] = act'(output) * output_grad, as the pair it is made of and as its value
  auto g_raw = [&](int row, int col) -> float2 {
    int const r = row < p.batch ? row : p.batch - 1, c = col < p.out_dim ? col : p.out_dim - 1;
    int64_t const i = (int64_t)r * p.out_dim + c;
    float yv = 0.0f;
    if constexpr (ACT == FFK_ACT_RELU || ACT == FFK_ACT_SIGMOID || ACT == FFK_ACT_TANH) yv = p.y[i];
    return make_float2(yv, p.dy[i]);
  };
  auto g_val = [&](float2 r) -> float { return small_act_grad<ACT>(p.relu_mode, r.x, r.y); };
  if (bid < p.tiles_dx) {
    // input_grad[batch, in] (+)= g[batch, out] . weight[out, in]
    int const nbn = (p.in_dim + 63) / 64;
    auto b = [&](int k, int n) -> float {
      return p.w[(int64_t)(k < p.out_dim ? k : p.out_dim - 1) * p.in_dim + (n < p.in_dim ? n : p.in_dim - 1)];
    };
    bool const add = (p.accumulate & FFK_ACC_INPUT) != 0;
    auto store = [&](int m, int n, float v) { p.dx[(int64_t)m * p.in_dim + n] = v; };
    small_f32_tile<true, false>(g_raw, g_val, b, p.batch, p.in_dim, p.out_dim, (bid / nbn) * 64, (bid % nbn) * 64, store, As, Bs,
                                add ? p.dx : nullptr, p.in_dim);
  } else if (bid < p.tiles_dx + p.tiles_dw) {
    // weight_grad[out, in] (+)= g[batch, out]^T . input[batch, in]
    int const tb = bid - p.tiles_dx, nbn = (p.in_dim + 63) / 64;
    auto a = [&](int m, int k) -> float2 { return g_raw(k, m); };
    auto b = [&](int k, int n) -> float {
      return p.x[(int64_t)(k < p.batch ? k : p.batch - 1) * p.in_dim + (n < p.in_dim ? n : p.in_dim - 1)];
    };
    bool const add = (p.accumulate & FFK_ACC_WEIGHT) != 0;
    auto store = [&](int m, int n, float v) { p.dw[(int64_t)m * p.in_dim + n] = v; };
    small_f32_tile<false, false>(a, g_val, b, p.out_dim, p.in_dim, p.batch, (tb / nbn) * 64, (tb % nbn) * 64, store, As, Bs,
                                add ? p.dw : nullptr, p.in_dim);
  } else {
    // bias_grad[out] (+)= column sums of g: 64 columns, four row lanes that meet in LDS
    int const col = (bid - p.tiles_dx - p.tiles_dw) * 64 + (threadIdx.x & 63);
    int const ry = threadIdx.x >> 6;
    float s = 0.0f;
    for (int row = ry; row < p.batch; row += 32) {  // eight loads in flight, added in row order
      float2 v[8];
#pragma unroll
      for (int i = 0; i < 8; i++) v[i] = g_raw(row + 4 * i, col);
#pragma unroll
      for (int i = 0; i < 8; i++) s += row + 4 * i < p.batch ? g_val(v[i]) : 0.0f;
    }
    As[ry][threadIdx.x & 63] = s;
    __syncthreads();
    if (ry == 0 && col < p.out_dim) {
      float const v = (As[0][threadIdx.x] + As[1][threadIdx.x]) + (As[2][threadIdx.x] + As[3][threadIdx.x]);
      p.db[col] = (p.accumulate & FFK_ACC_BIAS) != 0 ? p.db[col] + v : v;
    }
  }
}

// Forward of a small fp32 Linear: output = act(input . weight^T + bias), one 64x64 tile per
// workgroup, the same 64-deep reduction tiles.
struct SmallLinearFwd {
  float const *x, *w, *bias;
  float *y;
  int batch, in_dim, out_dim, act;
};

__global__ __launch_bounds__(256) void linear_small_fwd_f32_kernel(SmallLinearFwd p) {
  __shared__ float As[kSmallBK][68], Bs[kSmallBK][68];
  int const nbn = (p.out_dim + 63) / 64;
  auto a = [&](int m, int k) -> float {
    return p.x[(int64_t)(m < p.batch ? m : p.batch - 1) * p.in_dim + (k < p.in_dim ? k : p.in_dim - 1)];
  };
  // weight is [out, in]: b(k, n) = weight[n][k], k contiguous like the input's
  auto b = [&](int k, int n) -> float {
    return p.w[(int64_t)(n < p.out_dim ? n : p.out_dim - 1) * p.in_dim + (k < p.in_dim ? k : p.in_dim - 1)];
  };
  auto store = [&](int m, int n, float v) {
    v += p.bias != nullptr ? p.bias[n] : 0.0f;
    switch (p.act) {
      case FFK_ACT_RELU: v = v >= 0.0f ? v : 0.0f; break;  // tensor_accessor_unary_ops.cc:32-38 keeps x >= 0
      case FFK_ACT_SIGMOID: v = 1.0f / (1.0f + expf(-v)); break;
      case FFK_ACT_TANH: v = tanhf(v); break;
      case FFK_ACT_GELU: v = gelu_forward(v); break;
      default: break;
    }
    p.y[(int64_t)m * p.out_dim + n] = v;
  };
  small_f32_tile<true, true>(a, [](float v) { return v; }, b, p.batch, p.out_dim, p.in_dim, (blockIdx.x / nbn) * 64, (blockIdx.x % nbn) * 64, store, As, Bs);
}

// Small enough that launches, not work, set the time: at most two workgroups per CU in all.
static bool small_linear_bwd(int dtype, int64_t batch, int64_t in_dim, int64_t out_dim, bool bias, int &tiles_dx,
                             int &tiles_dw, int &blocks) {
  // a tile's reduction (out_dim for the input gradient, batch for the weight gradient) stays short
  if (dtype != FFK_FLOAT || batch > kSmallMaxDepth || out_dim > kSmallMaxDepth || in_dim > (1 << 20)) return false;
  int64_t const tdx = ceil_div(batch, 64) * ceil_div(in_dim, 64), tdw = ceil_div(out_dim, 64) * ceil_div(in_dim, 64);
  int64_t const tb = bias ? ceil_div(out_dim, 64) : 0;
  if (tdx + tdw + tb > 2 * kNumCU) return false;
  tiles_dx = (int)tdx;
  tiles_dw = (int)tdw;
  blocks = (int)(tdx + tdw + tb);
  return true;
}

}  // namespace ffk

using namespace ffk;

extern "C" size_t ffk_linear_backward_workspace_bytes(int dtype, int activation,
                                                      int use_bias,
                                                      int64_t batch,
                                                      int64_t out_dim) {
  size_t bytes = 0;
  if (activation != FFK_ACT_NONE) {
    bytes += align256((size_t)batch * (size_t)out_dim * dtype_size(dtype));
  }
  if (use_bias) {
    bytes += align256((size_t)colsum_partials_elems(batch, out_dim) * sizeof(float));
  }
  return bytes;
}

extern "C" int ffk_linear_forward(ffk_stream_t stream, int dtype,
                                  int activation, void const *input,
                                  void *output, void const *weight,
                                  void const *bias, int64_t batch,
                                  int64_t in_dim, int64_t out_dim) {
  FFK_REQUIRE(dtype == FFK_FLOAT || dtype == FFK_BF16,
              "linear_forward: dtype %d not supported", dtype);
  FFK_REQUIRE(activation >= FFK_ACT_NONE && activation <= FFK_ACT_GELU,
              "linear_forward: Unhandled activation function %d", activation);
  FFK_REQUIRE(batch > 0 && in_dim > 0 && out_dim > 0,
              "linear_forward: non-positive dimension");
  FFK_REQUIRE(input && output && weight, "linear_forward: NULL tensor");
  if (dtype == FFK_FLOAT && batch <= 8192 && ceil_div(batch, 64) * ceil_div(out_dim, 64) <= 2 * kNumCU &&
      in_dim <= kSmallMaxDepth) {
    SmallLinearFwd p = {static_cast<float const *>(input), static_cast<float const *>(weight),
                        static_cast<float const *>(bias), static_cast<float *>(output),
                        (int)batch, (int)in_dim, (int)out_dim, activation};
    unsigned const blocks = (unsigned)(ceil_div(batch, 64) * ceil_div(out_dim, 64));
    linear_small_fwd_f32_kernel<<<blocks, 256, 0, as_stream(stream)>>>(p);
    FFK_CHECK_LAUNCH();
    return FFK_OK;
  }
  GemmEpilogue ep;
  ep.bias = bias;
  ep.activation = activation;
  // output[batch,out] = input[batch,in] . weight[out,in]^T
  return gemm_dispatch(as_stream(stream), dtype, false, true, batch, out_dim,
                       in_dim, input, in_dim, weight, in_dim, output, out_dim, ep);
}

// input_tail: operators the input gradient passes through while it is written
// (GemmEpilogue's tail fields), or nullptr.
static int linear_backward_impl(
    ffk_stream_t stream, int dtype, int activation, int relu_grad_mode,
    void const *output, void const *output_grad, void const *input,
    void *input_grad, void const *weight, void *weight_grad, void *bias_grad,
    int64_t batch, int64_t in_dim, int64_t out_dim, void *workspace,
    size_t workspace_bytes, int accumulate, GemmEpilogue const *input_tail) {
  FFK_REQUIRE(dtype == FFK_FLOAT || dtype == FFK_BF16,
              "linear_backward: dtype %d not supported", dtype);
  FFK_REQUIRE(activation >= FFK_ACT_NONE && activation <= FFK_ACT_TANH,
              "linear_backward: Unhandled activation function %d (GELU needs "
              "the pre-activation; use an ElementUnary GELU op)",
              activation);
  FFK_REQUIRE(batch > 0 && in_dim > 0 && out_dim > 0,
              "linear_backward: non-positive dimension");
  FFK_REQUIRE(output_grad && weight && input, "linear_backward: NULL tensor");
  hipStream_t st = as_stream(stream);
  if (activation != FFK_ACT_NONE) {
    FFK_REQUIRE(output != nullptr, "linear_backward: output needed for activation");
  }
  // a small fp32 problem whose three gradients are all asked for: one launch, no scratch
  int tiles_dx = 0, tiles_dw = 0, blocks = 0;
  if (input_tail == nullptr && input_grad != nullptr && weight_grad != nullptr &&
      small_linear_bwd(dtype, batch, in_dim, out_dim, bias_grad != nullptr, tiles_dx, tiles_dw, blocks)) {
    SmallLinearBwd p;
    p.y = static_cast<float const *>(output);
    p.dy = static_cast<float const *>(output_grad);
    p.x = static_cast<float const *>(input);
    p.w = static_cast<float const *>(weight);
    p.dx = static_cast<float *>(input_grad);
    p.dw = static_cast<float *>(weight_grad);
    p.db = static_cast<float *>(bias_grad);
    p.batch = (int)batch;
    p.in_dim = (int)in_dim;
    p.out_dim = (int)out_dim;
    p.act = activation;
    p.relu_mode = relu_grad_mode;
    p.accumulate = accumulate;
    p.tiles_dx = tiles_dx;
    p.tiles_dw = tiles_dw;
    switch (activation) {
      case FFK_ACT_RELU: linear_small_bwd_f32_kernel<FFK_ACT_RELU><<<blocks, 256, 0, st>>>(p); break;
      case FFK_ACT_SIGMOID: linear_small_bwd_f32_kernel<FFK_ACT_SIGMOID><<<blocks, 256, 0, st>>>(p); break;
      case FFK_ACT_TANH: linear_small_bwd_f32_kernel<FFK_ACT_TANH><<<blocks, 256, 0, st>>>(p); break;
      default: linear_small_bwd_f32_kernel<FFK_ACT_NONE><<<blocks, 256, 0, st>>>(p); break;
    }
    FFK_CHECK_LAUNCH();
    return FFK_OK;
  }
  size_t need = ffk_linear_backward_workspace_bytes(dtype, activation,
                                                    bias_grad != nullptr, batch, out_dim);
  if (need > 0 && (workspace == nullptr || workspace_bytes < need)) {
    return fail(FFK_ERR_WORKSPACE,
                "linear_backward: workspace of %zu bytes needed, %zu given", need,
                workspace_bytes);
  }
  uint8_t *ws = static_cast<uint8_t *>(workspace);
  void const *g = output_grad;
  if (activation != FFK_ACT_NONE) {
    int64_t n = batch * out_dim;
    hipError_t e = dtype == FFK_FLOAT
                       ? act_grad<float>(st, activation, relu_grad_mode, output, output_grad, ws, n)
                       : act_grad<bf16>(st, activation, relu_grad_mode, output, output_grad, ws, n);
    FFK_HIP(e);
    g = ws;
    ws += align256((size_t)n * dtype_size(dtype));
  }
  GemmEpilogue ep;
  int rc;
  if (input_grad != nullptr) {
    GemmEpilogue dx = input_tail != nullptr ? *input_tail : ep;
    dx.accumulate = (accumulate & FFK_ACC_INPUT) != 0;
    // input_grad[batch,in] = g[batch,out] . weight[out,in]
    if (input_tail != nullptr &&
        !gemm_tail_supported(dtype, false, false, batch, in_dim, out_dim, g, out_dim, weight, in_dim,
                             input_grad, in_dim, dx)) {
      return FFK_ERR_UNSUPPORTED;  // before anything is launched: the caller runs the separate operators
    }
    rc = gemm_dispatch(st, dtype, false, false, batch, in_dim, out_dim, g, out_dim,
                       weight, in_dim, input_grad, in_dim, dx);
    if (rc != FFK_OK) return rc;
  }
  if (weight_grad != nullptr) {
    ep.accumulate = (accumulate & FFK_ACC_WEIGHT) != 0;
    // weight_grad[out,in] = g[batch,out]^T . input[batch,in]
    rc = gemm_dispatch(st, dtype, true, false, out_dim, in_dim, batch, g, out_dim,
                       input, in_dim, weight_grad, in_dim, ep);
    if (rc != FFK_OK) return rc;
  }
  if (bias_grad != nullptr) {
    rc = colsum_dispatch(st, dtype, g, out_dim, batch, out_dim, bias_grad,
                         (accumulate & FFK_ACC_BIAS) != 0, reinterpret_cast<float *>(ws));
    if (rc != FFK_OK) return rc;
  }
  return FFK_OK;
}

extern "C" int ffk_linear_backward(
    ffk_stream_t stream, int dtype, int activation, int relu_grad_mode,
    void const *output, void const *output_grad, void const *input,
    void *input_grad, void const *weight, void *weight_grad, void *bias_grad,
    int64_t batch, int64_t in_dim, int64_t out_dim, void *workspace,
    size_t workspace_bytes, int accumulate) {
  return linear_backward_impl(stream, dtype, activation, relu_grad_mode, output, output_grad, input,
                              input_grad, weight, weight_grad, bias_grad, batch, in_dim, out_dim,
                              workspace, workspace_bytes, accumulate, nullptr);
}

extern "C" int ffk_linear_l2_regularizer_grad(ffk_stream_t stream, int dtype, void const *weight,
                                              void *weight_grad, int64_t elems, float lambda) {
  FFK_REQUIRE(dtype == FFK_FLOAT || dtype == FFK_BF16, "linear_l2_regularizer_grad: dtype %d not supported", dtype);
  FFK_REQUIRE(weight && weight_grad, "linear_l2_regularizer_grad: NULL tensor");
  FFK_REQUIRE(elems > 0, "linear_l2_regularizer_grad: non-positive element count");
  hipStream_t st = as_stream(stream);
  FFK_HIP(dtype == FFK_FLOAT ? l2_reg_grad<float>(st, weight, weight_grad, elems, lambda)
                             : l2_reg_grad<bf16>(st, weight, weight_grad, elems, lambda));
  return FFK_OK;
}

namespace ffk {

int linear_gelu_dropout_forward(hipStream_t st, int dtype, void const *input, void *output,
                                void *dropped, void const *weight, void const *bias, int64_t batch,
                                int64_t in_dim, int64_t out_dim, float rate, uint64_t seed,
                                uint64_t offset) {
  FFK_REQUIRE(input && output && dropped && weight, "linear_gelu_dropout_forward: NULL tensor");
  FFK_REQUIRE(batch > 0 && in_dim > 0 && out_dim > 0, "linear_gelu_dropout_forward: non-positive dimension");
  GemmEpilogue ep;
  ep.bias = bias;
  ep.tail = GemmEpilogue::kTailGeluDropout;
  ep.tail_out = dropped;
  int const prc = make_dropout_params("linear_gelu_dropout_forward", rate, seed, offset, ep.tail_dropout);
  if (prc != FFK_OK) return prc;
  if (!gemm_tail_supported(dtype, false, true, batch, out_dim, in_dim, input, in_dim, weight, in_dim,
                           output, out_dim, ep)) {
    return FFK_ERR_UNSUPPORTED;
  }
  return gemm_dispatch(st, dtype, false, true, batch, out_dim, in_dim, input, in_dim, weight, in_dim,
                       output, out_dim, ep);
}

int linear_dropout_add_forward(hipStream_t st, int dtype, void const *input, void const *residual,
                               void *output, void const *weight, void const *bias, int64_t batch,
                               int64_t in_dim, int64_t out_dim, float rate, uint64_t seed,
                               uint64_t offset) {
  FFK_REQUIRE(input && residual && output && weight, "linear_dropout_add_forward: NULL tensor");
  FFK_REQUIRE(batch > 0 && in_dim > 0 && out_dim > 0, "linear_dropout_add_forward: non-positive dimension");
  GemmEpilogue ep;
  ep.bias = bias;
  ep.tail = GemmEpilogue::kTailDropoutAdd;
  ep.tail_in = residual;
  int const prc = make_dropout_params("linear_dropout_add_forward", rate, seed, offset, ep.tail_dropout);
  if (prc != FFK_OK) return prc;
  if (!gemm_tail_supported(dtype, false, true, batch, out_dim, in_dim, input, in_dim, weight, in_dim,
                           output, out_dim, ep)) {
    return FFK_ERR_UNSUPPORTED;
  }
  return gemm_dispatch(st, dtype, false, true, batch, out_dim, in_dim, input, in_dim, weight, in_dim,
                       output, out_dim, ep);
}

int linear_backward_dropout_gelu(hipStream_t st, int dtype, void const *output_grad, void const *input,
                                 void const *gelu_input, void *input_grad, void const *weight,
                                 void *weight_grad, void *bias_grad, int64_t batch, int64_t in_dim,
                                 int64_t out_dim, void *workspace, size_t workspace_bytes,
                                 int accumulate, float rate, uint64_t seed, uint64_t offset,
                                 void *input_grad_colsum, float *colsum_partials, bool colsum_accumulate) {
  FFK_REQUIRE(output_grad && input && gelu_input && input_grad && weight,
              "linear_backward_dropout_gelu: NULL tensor");
  FFK_REQUIRE(input_grad_colsum == nullptr || colsum_partials != nullptr,
              "linear_backward_dropout_gelu: column sums need scratch for their partial sums");
  FFK_REQUIRE((accumulate & FFK_ACC_INPUT) == 0,
              "linear_backward_dropout_gelu: the input gradient is stored, not added");
  GemmEpilogue tail;
  tail.tail = GemmEpilogue::kTailDropoutGeluGrad;
  tail.tail_in = gelu_input;
  tail.tail_colsum_partials = input_grad_colsum != nullptr ? colsum_partials : nullptr;
  int const prc = make_dropout_params("linear_backward_dropout_gelu", rate, seed, offset, tail.tail_dropout);
  if (prc != FFK_OK) return prc;
  int const rc = linear_backward_impl(st, dtype, FFK_ACT_NONE, 0, nullptr, output_grad, input, input_grad, weight,
                                      weight_grad, bias_grad, batch, in_dim, out_dim, workspace, workspace_bytes,
                                      accumulate, &tail);
  if (rc != FFK_OK || input_grad_colsum == nullptr) return rc;
  return colsum_finish(st, dtype, colsum_partials, batch, in_dim, input_grad_colsum, colsum_accumulate);
}

}  // namespace ffk

extern "C" int ffk_linear_gelu_dropout_forward(ffk_stream_t stream, int dtype, void const *input,
                                               void *output, void *dropped, void const *weight,
                                               void const *bias, int64_t batch, int64_t in_dim,
                                               int64_t out_dim, float rate, uint64_t seed,
                                               uint64_t offset) {
  int const rc = ffk::linear_gelu_dropout_forward(as_stream(stream), dtype, input, output, dropped, weight,
                                                  bias, batch, in_dim, out_dim, rate, seed, offset);
  if (rc == FFK_ERR_UNSUPPORTED) {
    return fail(FFK_ERR_UNSUPPORTED, "linear_gelu_dropout_forward: no fused kernel for this shape; "
                                     "run Linear, GELU and Dropout one after the other");
  }
  return rc;
}

extern "C" int ffk_linear_dropout_add_forward(ffk_stream_t stream, int dtype, void const *input,
                                              void const *residual, void *output, void const *weight,
                                              void const *bias, int64_t batch, int64_t in_dim,
                                              int64_t out_dim, float rate, uint64_t seed,
                                              uint64_t offset) {
  int const rc = ffk::linear_dropout_add_forward(as_stream(stream), dtype, input, residual, output, weight,
                                                 bias, batch, in_dim, out_dim, rate, seed, offset);
  if (rc == FFK_ERR_UNSUPPORTED) {
    return fail(FFK_ERR_UNSUPPORTED, "linear_dropout_add_forward: no fused kernel for this shape; "
                                     "run Linear, Dropout and the addition one after the other");
  }
  return rc;
}

extern "C" int ffk_linear_backward_dropout_gelu(
    ffk_stream_t stream, int dtype, void const *output_grad, void const *input, void const *gelu_input,
    void *input_grad, void const *weight, void *weight_grad, void *bias_grad, int64_t batch,
    int64_t in_dim, int64_t out_dim, void *workspace, size_t workspace_bytes, int accumulate,
    float rate, uint64_t seed, uint64_t offset) {
  int const rc = ffk::linear_backward_dropout_gelu(as_stream(stream), dtype, output_grad, input, gelu_input,
                                                   input_grad, weight, weight_grad, bias_grad, batch,
                                                   in_dim, out_dim, workspace, workspace_bytes,
                                                   accumulate, rate, seed, offset, nullptr, nullptr, false);
  if (rc == FFK_ERR_UNSUPPORTED) {
    return fail(FFK_ERR_UNSUPPORTED, "linear_backward_dropout_gelu: no fused kernel for this shape; "
                                     "run Linear backward, Dropout backward and GELU backward one after the other");
  }
  return rc;
}

extern "C" size_t ffk_dropout_backward_bias_grad_workspace_bytes(int64_t batch, int64_t out_dim) {
  return align256((size_t)colsum_partials_elems(batch, out_dim) * sizeof(float));
}

extern "C" int ffk_dropout_backward_bias_grad(ffk_stream_t stream, int dtype, void const *output_grad,
                                              void *input_grad, int64_t batch, int64_t out_dim, void *bias_grad,
                                              int accumulate_bias, void *workspace, size_t workspace_bytes,
                                              float rate, uint64_t seed, uint64_t offset) {
  FFK_REQUIRE(output_grad && input_grad && bias_grad, "dropout_backward_bias_grad: NULL tensor");
  FFK_REQUIRE(batch > 0 && out_dim > 0, "dropout_backward_bias_grad: non-positive dimension");
  size_t const need = ffk_dropout_backward_bias_grad_workspace_bytes(batch, out_dim);
  if (workspace == nullptr || workspace_bytes < need) {
    return fail(FFK_ERR_WORKSPACE, "dropout_backward_bias_grad: workspace of %zu bytes needed, %zu given", need,
                workspace_bytes);
  }
  DropoutParams dp;
  int const prc = make_dropout_params("dropout_backward_bias_grad", rate, seed, offset, dp);
  if (prc != FFK_OK) return prc;
  int const rc = dropout_backward_colsum(as_stream(stream), dtype, output_grad, input_grad, batch, out_dim, bias_grad,
                                         accumulate_bias != 0, static_cast<float *>(workspace), dp);
  if (rc == FFK_ERR_UNSUPPORTED) {
    return fail(FFK_ERR_UNSUPPORTED, "dropout_backward_bias_grad: no fused kernel for this shape; run Dropout "
                                     "backward and let the Linear's backward sum its bias gradient");
  }
  return rc;
}

extern "C" int ffk_linear_backward_dropout_gelu_bias_grad(
    ffk_stream_t stream, int dtype, void const *output_grad, void const *input, void const *gelu_input,
    void *input_grad, void const *weight, void *weight_grad, void *bias_grad, int64_t batch, int64_t in_dim,
    int64_t out_dim, void *workspace, size_t workspace_bytes, int accumulate, float rate, uint64_t seed,
    uint64_t offset, void *gelu_bias_grad, int accumulate_gelu_bias, void *gelu_bias_workspace,
    size_t gelu_bias_workspace_bytes) {
  FFK_REQUIRE(gelu_bias_grad != nullptr, "linear_backward_dropout_gelu_bias_grad: NULL bias gradient");
  size_t const need = ffk_dropout_backward_bias_grad_workspace_bytes(batch, in_dim);
  if (gelu_bias_workspace == nullptr || gelu_bias_workspace_bytes < need) {
    return fail(FFK_ERR_WORKSPACE, "linear_backward_dropout_gelu_bias_grad: workspace of %zu bytes needed for the "
                                   "column sums, %zu given", need, gelu_bias_workspace_bytes);
  }
  int const rc = ffk::linear_backward_dropout_gelu(as_stream(stream), dtype, output_grad, input, gelu_input, input_grad,
                                                   weight, weight_grad, bias_grad, batch, in_dim, out_dim, workspace,
                                                   workspace_bytes, accumulate, rate, seed, offset, gelu_bias_grad,
                                                   static_cast<float *>(gelu_bias_workspace), accumulate_gelu_bias != 0);
  if (rc == FFK_ERR_UNSUPPORTED) {
    return fail(FFK_ERR_UNSUPPORTED, "linear_backward_dropout_gelu_bias_grad: no fused kernel for this shape; "
                                     "use ffk_linear_backward_dropout_gelu and let the first Linear's backward sum "
                                     "its bias gradient");
  }
  return rc;
}
