// LayerNorm forward/backward for gfx950: one pass over the data.
//
// forward : a row lives in the registers of one wavefront (or one workgroup
//           for long rows); mean and variance are reduced with wave shuffles,
//           the normalised row is written once.  (Reference: two kernels and
//           three reads of X, lib/kernels/src/cuda/ops/layer_norm_kernels.cu:
//           69-112,328-352.)
// backward: one pass over dY and X produces dX (the formula of
//           LayerNormBackwardCUDAKenrel, layer_norm_kernels.cu:163-181, which
//           the reference never launches) and per-workgroup partial column
//           sums for dgamma/dbeta, reduced by a second small kernel
//           (reference: ComputeInternalGradients + GammaBetaBackward, two more
//           passes, :115-290,354-410).
#include "rowwise.h"
#include "colreduce.h"
#include "fused_ops.h"
#include "dropout_rng.h"
#include <mutex>

namespace ffk {

// PRE: the row normalised is residual + dropout(X), computed here, rounded to T where the two
// separate operators would have stored it, and written to `summed` as well.
template <typename T, int EPT, int WPR, bool PRE = false, bool STREAM = false>
__global__ __launch_bounds__(kRowThreads) void layer_norm_fwd_kernel(
    T const *__restrict__ X, T *__restrict__ Y, T const *__restrict__ gamma,
    T const *__restrict__ beta, float *__restrict__ mean,
    float *__restrict__ rstd, int64_t M, int N, float eps,
    T const *__restrict__ residual = nullptr, T *__restrict__ summed = nullptr,
    DropoutParams drop = DropoutParams{}) {
  constexpr int V = VecIO<T>::kVec;
  constexpr int RPB = 4 / WPR;  // rows per workgroup
  constexpr int LANES = 64 * WPR;
  __shared__ float smem[2][4][2];
  RowReducer<WPR> red(smem);
  int const nvec = N / V;
  int const lane = WPR == 1 ? (threadIdx.x & 63) : threadIdx.x;
  int64_t const row = (int64_t)blockIdx.x * RPB + (WPR == 1 ? (threadIdx.x >> 6) : 0);
  bool const row_ok = row < M;
  T const *xr = X + (row_ok ? row : 0) * (int64_t)N;

  float x[EPT][V];
  float s = 0.0f;
  // Short rows (up to two vectors per lane): gamma and beta are asked for before the row's two
  // reductions, not after them: such a kernel is one chain of memory round trips, and this one
  // then runs under the others.  Longer rows load them where they are used; their registers
  // are better spent on resident waves.
  constexpr bool kEarly = EPT <= 2;
  float g[EPT][V], b[EPT][V];
  auto load_params = [&](int j) __attribute__((always_inline)) {
    int v = lane + j * LANES;
#pragma unroll
    for (int e = 0; e < V; e++) {
      g[j][e] = 1.0f;
      b[j][e] = 0.0f;
    }
    if (v < nvec) {
      if (gamma != nullptr) VecIO<T>::load(gamma + (int64_t)v * V, g[j]);
      if (beta != nullptr) VecIO<T>::load(beta + (int64_t)v * V, b[j]);
    }
  };
  if constexpr (kEarly) {
#pragma unroll
    for (int j = 0; j < EPT; j++) load_params(j);
  }
#pragma unroll
  for (int j = 0; j < EPT; j++) {
    int v = lane + j * LANES;
    if (v < nvec) {
      if (STREAM) {
        VecIO<T>::load_stream(xr + (int64_t)v * V, x[j]);
      } else {
        VecIO<T>::load(xr + (int64_t)v * V, x[j]);
      }
      if constexpr (PRE) {
        static_assert(V == 4 || V == 8, "a lane's vector is a Philox block or half of one");
        if (row_ok) {
          int64_t const at = row * (int64_t)N + (int64_t)v * V;
          float r[V];
          VecIO<T>::load(residual + at, r);
          uint64_t const e0 = drop.offset + (uint64_t)at;
          uint32_t w[4];
          philox4x32_10(e0 >> 3, drop.key, w);
          if (V == 4 && (e0 & 4)) {
            w[0] = w[2];
            w[1] = w[3];
          }
#pragma unroll
          for (int e = 0; e < V; e++) {
            float const d = keep(w, e, drop) ? x[j][e] * drop.scale : 0.0f;
            x[j][e] = storage_round<T>(storage_round<T>(d) + r[e]);
          }
          VecIO<T>::store(summed + at, x[j]);
        }
      }
#pragma unroll
      for (int e = 0; e < V; e++) s += x[j][e];
    } else {
#pragma unroll
      for (int e = 0; e < V; e++) x[j][e] = 0.0f;
    }
  }
  float const inv_n = 1.0f / (float)N;
  float const mu = red.sum(s) * inv_n;
  float q = 0.0f;
#pragma unroll
  for (int j = 0; j < EPT; j++) {
    int v = lane + j * LANES;
    if (v < nvec) {
#pragma unroll
      for (int e = 0; e < V; e++) {
        float d = x[j][e] - mu;
        q += d * d;
      }
    }
  }
  float const var = red.sum(q) * inv_n;
  float const rs = 1.0f / sqrtf(var + eps);
  if (!row_ok) return;
  if (lane == 0) {
    mean[row] = mu;
    rstd[row] = rs;
  }
  T *yr = Y + row * (int64_t)N;
#pragma unroll
  for (int j = 0; j < EPT; j++) {
    int v = lane + j * LANES;
    if (v < nvec) {
      float y[V];
      if constexpr (!kEarly) load_params(j);
#pragma unroll
      for (int e = 0; e < V; e++) {
        float xh = (x[j][e] - mu) * rs;
        y[e] = xh * g[j][e] + b[j][e];
      }
      if (STREAM) {
        VecIO<T>::store_stream(yr + (int64_t)v * V, y);
      } else {
        VecIO<T>::store(yr + (int64_t)v * V, y);
      }
    }
  }
}

// Generic forward: any N, one workgroup per row, scalar accesses.
template <typename T>
__global__ __launch_bounds__(kRowThreads) void layer_norm_fwd_generic_kernel(
    T const *__restrict__ X, T *__restrict__ Y, T const *__restrict__ gamma,
    T const *__restrict__ beta, float *__restrict__ mean,
    float *__restrict__ rstd, int64_t M, int N, float eps) {
  __shared__ float smem[2][4][2];
  RowReducer<4> red(smem);
  int64_t const row = blockIdx.x;
  T const *xr = X + row * (int64_t)N;
  float s = 0.0f;
  for (int j = threadIdx.x; j < N; j += kRowThreads) s += VecIO<T>::load1(xr + j);
  float const mu = red.sum(s) / (float)N;
  float q = 0.0f;
  for (int j = threadIdx.x; j < N; j += kRowThreads) {
    float d = VecIO<T>::load1(xr + j) - mu;
    q += d * d;
  }
  float const rs = 1.0f / sqrtf(red.sum(q) / (float)N + eps);
  if (threadIdx.x == 0) {
    mean[row] = mu;
    rstd[row] = rs;
  }
  T *yr = Y + row * (int64_t)N;
  for (int j = threadIdx.x; j < N; j += kRowThreads) {
    float gv = gamma != nullptr ? VecIO<T>::load1(gamma + j) : 1.0f;
    float bv = beta != nullptr ? VecIO<T>::load1(beta + j) : 0.0f;
    VecIO<T>::store1(yr + j, (VecIO<T>::load1(xr + j) - mu) * rs * gv + bv);
  }
}

// Backward, persistent over rows so that the dgamma/dbeta partial sums stay
// in registers until the workgroup is done.
// DROP: dropout_backward(dX as stored) is written to `dropped` as well (the gradient entering
// a dropout whose output fed the residual sum that this LayerNorm normalised).
template <typename T, int EPT, int WPR, bool ACC, bool DROP = false>
__global__ __launch_bounds__(kRowThreads) void layer_norm_bwd_kernel(
    T const *__restrict__ dY, T const *__restrict__ X,
    float const *__restrict__ mean, float const *__restrict__ rstd,
    T const *__restrict__ gamma, T *dX, float *__restrict__ partials,
    int64_t M, int N, T const *res, T *__restrict__ dropped = nullptr,
    DropoutParams drop = DropoutParams{}, bool stream_out = false, bool round_first = true) {
  // stream_out: dX is too large to be found in cache by its reader; store it past the caches.
  // ACC with res == nullptr: dX += gradient (one rounding).  ACC with res set and round_first:
  // dX = res + gradient rounded to the storage type, i.e. what a separate element-wise add of
  // res to the stored gradient would give; without round_first the sum is rounded once, i.e.
  // what dX += gradient gives when dX holds a copy of res.
  constexpr int V = VecIO<T>::kVec;
  constexpr int RPB = 4 / WPR;
  constexpr int LANES = 64 * WPR;
  __shared__ float smem[2][4][2];
  RowReducer<WPR> red(smem);
  int const nvec = N / V;
  int const lane = WPR == 1 ? (threadIdx.x & 63) : threadIdx.x;
  int const sub = WPR == 1 ? (threadIdx.x >> 6) : 0;
  float const inv_n = 1.0f / (float)N;

  float g[EPT][V], dg[EPT][V], db[EPT][V];
#pragma unroll
  for (int j = 0; j < EPT; j++) {
    int v = lane + j * LANES;
#pragma unroll
    for (int e = 0; e < V; e++) {
      g[j][e] = 1.0f;
      dg[j][e] = 0.0f;
      db[j][e] = 0.0f;
    }
    if (gamma != nullptr && v < nvec) {
      VecIO<T>::load(gamma + (int64_t)v * V, g[j]);
    }
  }

  int64_t const row_step = (int64_t)gridDim.x * RPB;
  // Two row buffers used in turn: the loads of the next row are issued into the other buffer
  // as soon as this row is unpacked, so they are in flight while this row is reduced.  (A
  // third buffer, two rows ahead, measured 2% slower: the kernel is short of neither requests
  // nor latency cover.)
  // Lanes past the row's end never load: their registers keep these zeros, which add nothing
  // to any sum, so the arithmetic below needs no bounds checks.
  u32x4 rxa[EPT], rdya[EPT], rxb[EPT], rdyb[EPT];
#pragma unroll
  for (int j = 0; j < EPT; j++) {
    rxa[j] = rdya[j] = rxb[j] = rdyb[j] = u32x4{0, 0, 0, 0};
  }
  // A wave whose row lies past the end (the last workgroup's spare waves) gets zeros, which
  // leave dgamma / dbeta as they are.
  auto issue_row = [&](u32x4 (&rx)[EPT], u32x4 (&rdy)[EPT], int64_t base) {
    int64_t const r = base + sub;
    if (r < M) {
#pragma unroll
      for (int j = 0; j < EPT; j++) {
        int v = lane + j * LANES;
        if (v < nvec) {
          rx[j] = load_raw_stream(X + r * (int64_t)N + (int64_t)v * V);
          rdy[j] = load_raw_stream(dY + r * (int64_t)N + (int64_t)v * V);
        }
      }
    } else {
#pragma unroll
      for (int j = 0; j < EPT; j++) {
        rx[j] = u32x4{0, 0, 0, 0};
        rdy[j] = u32x4{0, 0, 0, 0};
      }
    }
  };
  // One row from the buffers (rx, rdy); the next row goes into (ox, ody).  Every wave of a workgroup runs the same number of rows so the barriers
  // inside the reducer stay aligned.
  auto do_row = [&](u32x4 (&rx)[EPT], u32x4 (&rdy)[EPT], u32x4 (&ox)[EPT], u32x4 (&ody)[EPT], int64_t base) {
    int64_t const row = base + sub;
    bool const row_ok = row < M;
    int64_t const r = row_ok ? row : M - 1;
    float x[EPT][V], dy[EPT][V];
    float const mu = mean[r], rs = rstd[r];
    float s1 = 0.0f, s2 = 0.0f;  // sum dy*g, sum dy*g*xhat
#pragma unroll
    for (int j = 0; j < EPT; j++) {
      unpack_raw(rx[j], x[j], (T const *)nullptr);
      unpack_raw(rdy[j], dy[j], (T const *)nullptr);
    }
    if (base + row_step < M) issue_row(ox, ody, base + row_step);
#pragma unroll
    for (int j = 0; j < EPT; j++) {
#pragma unroll
      for (int e = 0; e < V; e++) {
        float xh = (x[j][e] - mu) * rs;
        float const dyv = dy[j][e];
        float dyg = dyv * g[j][e];
        s1 += dyg;
        s2 += dyg * xh;
        x[j][e] = xh;
        dg[j][e] += dyv * xh;
        db[j][e] += dyv;
        dy[j][e] = dyg;
      }
    }
    red.sum2(s1, s2);
    // rs * (dy g - m1 - xhat m2) as two fused operations per element
    float const c0 = -(s1 * inv_n) * rs, c1 = -(s2 * inv_n) * rs;
    if (row_ok && dX != nullptr) {
#pragma unroll
      for (int j = 0; j < EPT; j++) {
        int v = lane + j * LANES;
        if (v < nvec) {
          float o[V];
          T *dst = dX + row * (int64_t)N + (int64_t)v * V;
          if (ACC) {
            VecIO<T>::load(res != nullptr ? res + row * (int64_t)N + (int64_t)v * V : dst, o);
          }
#pragma unroll
          for (int e = 0; e < V; e++) {
            float val = fmaf(dy[j][e], rs, fmaf(x[j][e], c1, c0));
            if (ACC && res != nullptr && round_first) val = storage_round<T>(val);
            o[e] = ACC ? o[e] + val : val;
          }
          if (stream_out) {
            VecIO<T>::store_stream(dst, o);
          } else {
            VecIO<T>::store(dst, o);
          }
          if constexpr (DROP) {
            static_assert(V == 4 || V == 8, "a lane's vector is a Philox block or half of one");
            int64_t const at = row * (int64_t)N + (int64_t)v * V;
            uint64_t const e0 = drop.offset + (uint64_t)at;
            uint32_t w[4];
            philox4x32_10(e0 >> 3, drop.key, w);
            if (V == 4 && (e0 & 4)) {
              w[0] = w[2];
              w[1] = w[3];
            }
#pragma unroll
            for (int e = 0; e < V; e++) o[e] = keep(w, e, drop) ? storage_round<T>(o[e]) * drop.scale : 0.0f;
            VecIO<T>::store(dropped + at, o);
          }
        }
      }
    }
  };
  {
    int64_t base = (int64_t)blockIdx.x * RPB;
    if (base < M) issue_row(rxa, rdya, base);
    while (base < M) {
      do_row(rxa, rdya, rxb, rdyb, base);
      base += row_step;
      if (base >= M) break;
      do_row(rxb, rdyb, rxa, rdya, base);
      base += row_step;
    }
  }

  // Workgroup partial: with WPR == 1 the four waves hold different rows of the
  // same columns; fold them through LDS first.
  float *pg = partials + (int64_t)blockIdx.x * 2 * N;
  float *pb = pg + N;
  if (WPR == 1) {
    __shared__ float fold[3][64][V + 1];
#pragma unroll
    for (int j = 0; j < EPT; j++) {
      int v = lane + j * LANES;
      for (int pass = 0; pass < 2; pass++) {
        __syncthreads();
        if (sub > 0) {
#pragma unroll
          for (int e = 0; e < V; e++) {
            fold[sub - 1][lane][e] = pass == 0 ? dg[j][e] : db[j][e];
          }
        }
        __syncthreads();
        if (sub == 0 && v < nvec) {
#pragma unroll
          for (int e = 0; e < V; e++) {
            float tot = (pass == 0 ? dg[j][e] : db[j][e]) + fold[0][lane][e] +
                        fold[1][lane][e] + fold[2][lane][e];
            (pass == 0 ? pg : pb)[(int64_t)v * V + e] = tot;
          }
        }
      }
    }
  } else {
#pragma unroll
    for (int j = 0; j < EPT; j++) {
      int v = lane + j * LANES;
      if (v < nvec) {
#pragma unroll
        for (int e = 0; e < V; e++) {
          pg[(int64_t)v * V + e] = dg[j][e];
          pb[(int64_t)v * V + e] = db[j][e];
        }
      }
    }
  }
}

// Generic backward: any N; one workgroup per row for dX, then a column kernel
// for dgamma/dbeta that walks all rows (GammaBetaBackwardSimpleCUDAKernel
// style, layer_norm_kernels.cu:184-214).
template <typename T>
__global__ __launch_bounds__(kRowThreads) void layer_norm_bwd_generic_dx_kernel(
    T const *__restrict__ dY, T const *__restrict__ X,
    float const *__restrict__ mean, float const *__restrict__ rstd,
    T const *__restrict__ gamma, T *dX, int64_t M, int N, int acc) {
  __shared__ float smem[2][4][2];
  RowReducer<4> red(smem);
  int64_t const row = blockIdx.x;
  float const mu = mean[row], rs = rstd[row];
  float s1 = 0.0f, s2 = 0.0f;
  for (int j = threadIdx.x; j < N; j += kRowThreads) {
    float gv = gamma != nullptr ? VecIO<T>::load1(gamma + j) : 1.0f;
    float dyg = VecIO<T>::load1(dY + row * (int64_t)N + j) * gv;
    float xh = (VecIO<T>::load1(X + row * (int64_t)N + j) - mu) * rs;
    s1 += dyg;
    s2 += dyg * xh;
  }
  red.sum2(s1, s2);
  float const m1 = s1 / (float)N, m2 = s2 / (float)N;
  for (int j = threadIdx.x; j < N; j += kRowThreads) {
    float gv = gamma != nullptr ? VecIO<T>::load1(gamma + j) : 1.0f;
    float dyg = VecIO<T>::load1(dY + row * (int64_t)N + j) * gv;
    float xh = (VecIO<T>::load1(X + row * (int64_t)N + j) - mu) * rs;
    float val = rs * (dyg - m1 - xh * m2);
    T *dst = dX + row * (int64_t)N + j;
    if (acc) val += VecIO<T>::load1(dst);
    VecIO<T>::store1(dst, val);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void layer_norm_bwd_generic_param_kernel(
    T const *__restrict__ dY, T const *__restrict__ X,
    float const *__restrict__ mean, float const *__restrict__ rstd, T *dgamma,
    T *dbeta, int64_t M, int N, int acc) {
  int const j = blockIdx.x * 256 + threadIdx.x;
  if (j >= N) return;
  float sg = 0.0f, sb = 0.0f;
  for (int64_t i = 0; i < M; i++) {
    float d = VecIO<T>::load1(dY + i * (int64_t)N + j);
    float xh = (VecIO<T>::load1(X + i * (int64_t)N + j) - mean[i]) * rstd[i];
    sg += d * xh;
    sb += d;
  }
  if (dgamma != nullptr) VecIO<T>::store1(dgamma + j, acc ? sg + VecIO<T>::load1(dgamma + j) : sg);
  if (dbeta != nullptr) VecIO<T>::store1(dbeta + j, acc ? sb + VecIO<T>::load1(dbeta + j) : sb);
}

// Two workgroups per CU: with one the memory pipe runs short of requests (102 against 76 us on
// [16384, 4096] bf16), with three or four every workgroup's partial sums (2 N floats) and the
// kernel that adds them up cost more than the extra requests in flight gain (80 and 92 us).
constexpr int kLnBwdMaxBlocks = 2 * kNumCU;

static int ln_bwd_blocks(int64_t M, int wpr) {
  int64_t rpb = 4 / wpr;
  int64_t b = ceil_div(M, rpb);
  return (int)(b < kLnBwdMaxBlocks ? b : kLnBwdMaxBlocks);
}

template <typename T>
static int ln_forward(hipStream_t st, void const *x, void *y, void const *gamma,
                      void const *beta, float *mean, float *rstd, int64_t M,
                      int64_t N, float eps) {
  constexpr int V = VecIO<T>::kVec;
  T const *X = static_cast<T const *>(x);
  T *Y = static_cast<T *>(y);
  T const *G = static_cast<T const *>(gamma);
  T const *Bt = static_cast<T const *>(beta);
  int ept = 0, wpr = 0;
  bool vec = (N % V == 0) && aligned16(x) && aligned16(y) &&
             (gamma == nullptr || aligned16(gamma)) &&
             (beta == nullptr || aligned16(beta)) &&
             pick_row_config_small(N / V, ept, wpr);
  if (vec) {
    int64_t blocks = ceil_div(M, 4 / wpr);
    bool const stream = stream_past_caches(M * N, sizeof(T));
#define CALL(E, W)                                                             \
  do {                                                                         \
    if (stream)                                                                \
      layer_norm_fwd_kernel<T, E, W, false, true><<<(unsigned)blocks, kRowThreads, 0, st>>>( \
          X, Y, G, Bt, mean, rstd, M, (int)N, eps);                            \
    else                                                                       \
      layer_norm_fwd_kernel<T, E, W><<<(unsigned)blocks, kRowThreads, 0, st>>>( \
          X, Y, G, Bt, mean, rstd, M, (int)N, eps);                            \
  } while (0)
    FFK_ROW_DISPATCH_SMALL(ept, wpr, CALL);
#undef CALL
  } else {
    layer_norm_fwd_generic_kernel<T><<<(unsigned)M, kRowThreads, 0, st>>>(
        X, Y, G, Bt, mean, rstd, M, (int)N, eps);
  }
  FFK_CHECK_LAUNCH();
  return FFK_OK;
}

template <typename T>
static int ln_backward(hipStream_t st, void const *dy, void const *x,
                       float const *mean, float const *rstd, void const *gamma,
                       void *dx, void *dgamma, void *dbeta, int64_t M, int64_t N,
                       void *workspace, size_t workspace_bytes, bool acc,
                       void const *residual = nullptr, void *dropped = nullptr,
                       DropoutParams const *drop = nullptr, bool fit_blocks_to_workspace = false,
                       bool acc_params = false, bool round_first = true) {
  constexpr int V = VecIO<T>::kVec;
  T const *RES = static_cast<T const *>(residual);
  if (RES != nullptr) acc = true;
  if (dropped != nullptr && (RES == nullptr || dx == nullptr || N % 8 != 0 || (drop->offset & 7) != 0 || !aligned16(dropped))) {
    return fail(FFK_ERR_UNSUPPORTED, "layer_norm_backward: the dropped copy needs the residual form and whole Philox blocks");
  }
  T const *DY = static_cast<T const *>(dy);
  T const *X = static_cast<T const *>(x);
  T const *G = static_cast<T const *>(gamma);
  T *DX = static_cast<T *>(dx);
  int ept = 0, wpr = 0;
  bool vec = (N % V == 0) && aligned16(dy) && aligned16(x) &&
             (dx == nullptr || aligned16(dx)) && aligned16(residual) &&
             (gamma == nullptr || aligned16(gamma)) && pick_row_config_small(N / V, ept, wpr);
  if (!vec && RES != nullptr) {
    return fail(FFK_ERR_UNSUPPORTED, "layer_norm_backward: residual form needs the vector kernel");
  }
  if (vec) {
    int blocks = ln_bwd_blocks(M, wpr);
    size_t const per_block = 2 * (size_t)N * sizeof(float);
    if (fit_blocks_to_workspace && workspace_bytes / per_block < (size_t)blocks) {
      // fewer, longer-running workgroups: dX is unchanged, the parameter
      // gradients are summed over fewer partial rows
      blocks = (int)(workspace_bytes / per_block);
    }
    size_t need = (size_t)blocks * per_block;
    if (workspace == nullptr || blocks < 1 || workspace_bytes < need) {
      return fail(FFK_ERR_WORKSPACE,
                  "layer_norm_backward: workspace of %zu bytes needed, %zu given",
                  need, workspace_bytes);
    }
    float *partials = static_cast<float *>(workspace);
    bool const stream = stream_past_caches(M * N, sizeof(T));
#define CALL(E, W)                                                             \
  do {                                                                         \
    if (dropped != nullptr) {                                                  \
      if constexpr (sizeof(T) == 2)                                            \
        layer_norm_bwd_kernel<T, E, W, true, true><<<blocks, kRowThreads, 0, st>>>( \
            DY, X, mean, rstd, G, DX, partials, M, (int)N, RES,                \
            static_cast<T *>(dropped), *drop, stream, round_first);            \
    } else if (acc)                                                            \
      layer_norm_bwd_kernel<T, E, W, true><<<blocks, kRowThreads, 0, st>>>(    \
          DY, X, mean, rstd, G, DX, partials, M, (int)N, RES, nullptr, DropoutParams{}, stream, round_first); \
    else                                                                       \
      layer_norm_bwd_kernel<T, E, W, false><<<blocks, kRowThreads, 0, st>>>(   \
          DY, X, mean, rstd, G, DX, partials, M, (int)N, nullptr, nullptr, DropoutParams{}, stream); \
  } while (0)
    FFK_ROW_DISPATCH_SMALL(ept, wpr, CALL);
#undef CALL
    FFK_CHECK_LAUNCH();
    if (dgamma != nullptr || dbeta != nullptr) {
      // partials are [blocks][2][N]: gamma sums in columns [0, N), beta after
      FFK_HIP(colreduce_launch<T>(st, partials, blocks, (int)(2 * N), (int)N,
                                  static_cast<T *>(dgamma), static_cast<T *>(dbeta), acc_params));
      FFK_CHECK_LAUNCH();
    }
  } else {
    if (dx != nullptr) {
      layer_norm_bwd_generic_dx_kernel<T><<<(unsigned)M, kRowThreads, 0, st>>>(
          DY, X, mean, rstd, G, DX, M, (int)N, acc);
      FFK_CHECK_LAUNCH();
    }
    if (dgamma != nullptr || dbeta != nullptr) {
      layer_norm_bwd_generic_param_kernel<T>
          <<<(unsigned)ceil_div(N, 256), 256, 0, st>>>(
              DY, X, mean, rstd, static_cast<T *>(dgamma),
              static_cast<T *>(dbeta), M, (int)N, acc_params ? 1 : 0);
      FFK_CHECK_LAUNCH();
    }
  }
  return FFK_OK;
}

template <typename T>
static int ln_forward_pre(hipStream_t st, void const *in, void const *residual, void *summed, void *y,
                          void const *gamma, void const *beta, float *mean, float *rstd, int64_t M, int64_t N,
                          float eps, DropoutParams const &drop) {
  constexpr int V = VecIO<T>::kVec;
  int ept = 0, wpr = 0;
  bool vec = (N % 8 == 0) && (drop.offset & 7) == 0 && aligned16(in) && aligned16(residual) && aligned16(summed) &&
             aligned16(y) && (gamma == nullptr || aligned16(gamma)) && (beta == nullptr || aligned16(beta)) &&
             pick_row_config_small(N / V, ept, wpr);
  if (!vec) return FFK_ERR_UNSUPPORTED;
  int64_t blocks = ceil_div(M, 4 / wpr);
#define CALL(E, W)                                                                                  \
  layer_norm_fwd_kernel<T, E, W, true><<<(unsigned)blocks, kRowThreads, 0, st>>>(                  \
      static_cast<T const *>(in), static_cast<T *>(y), static_cast<T const *>(gamma),             \
      static_cast<T const *>(beta), mean, rstd, M, (int)N, eps, static_cast<T const *>(residual), \
      static_cast<T *>(summed), drop)
  FFK_ROW_DISPATCH_SMALL(ept, wpr, CALL);
#undef CALL
  FFK_CHECK_LAUNCH();
  return FFK_OK;
}

int dropout_add_layer_norm_forward(hipStream_t st, int dtype, void const *in, void const *residual,
                                   void *summed, void *y, void const *gamma, void const *beta,
                                   float *mean, float *rstd, int64_t M, int64_t N, float eps,
                                   float rate, uint64_t seed, uint64_t offset) {
  FFK_REQUIRE(M > 0 && N > 0 && M < (1ll << 31) && N < (1ll << 31), "dropout_add_layer_norm: bad shape");
  FFK_REQUIRE(in && residual && summed && y && mean && rstd, "dropout_add_layer_norm: NULL tensor");
  DropoutParams drop;
  int rc = make_dropout_params("dropout_add_layer_norm", rate, seed, offset, drop);
  if (rc != FFK_OK) return rc;
  // bf16 only: the one caller (the encoder-layer entry points) has no other type
  if (dtype == FFK_BF16) return ln_forward_pre<bf16>(st, in, residual, summed, y, gamma, beta, mean, rstd, M, N, eps, drop);
  return FFK_ERR_UNSUPPORTED;
}

int layer_norm_backward_add_residual(hipStream_t st, int dtype, void const *dy,
                                     void const *x, float const *mean,
                                     float const *rstd, void const *gamma,
                                     void const *residual, void *dx,
                                     void *dgamma, void *dbeta, int64_t M,
                                     int64_t N, void *workspace,
                                     size_t workspace_bytes, void *dropped,
                                     float rate, uint64_t seed, uint64_t offset, bool acc_params,
                                     bool round_first) {
  FFK_REQUIRE(M > 0 && N > 0 && M < (1ll << 31) && N < (1ll << 31),
              "layer_norm_backward: bad shape");
  FFK_REQUIRE(dy && x && mean && rstd && residual && dx, "layer_norm_backward: NULL tensor");
  DropoutParams drop;
  if (dropped != nullptr) {
    int rc = make_dropout_params("layer_norm_backward", rate, seed, offset, drop);
    if (rc != FFK_OK) return rc;
  }
  if (dtype == FFK_FLOAT && dropped != nullptr) return FFK_ERR_UNSUPPORTED;  // the dropped copy is bf16 only
  if (dtype == FFK_FLOAT)
    return ln_backward<float>(st, dy, x, mean, rstd, gamma, dx, dgamma, dbeta, M, N,
                              workspace, workspace_bytes, true, residual, nullptr, nullptr, false, acc_params, round_first);
  if (dtype == FFK_BF16)
    return ln_backward<bf16>(st, dy, x, mean, rstd, gamma, dx, dgamma, dbeta, M, N,
                             workspace, workspace_bytes, true, residual, dropped, &drop, false, acc_params, round_first);
  return fail(FFK_ERR_UNSUPPORTED, "layer_norm_backward: dtype %d not supported", dtype);
}

}  // namespace ffk

using namespace ffk;

extern "C" int ffk_layer_norm_forward(ffk_stream_t stream, int dtype,
                                      void const *input, void *output,
                                      void const *gamma, void const *beta,
                                      float *mean, float *rstd, int64_t M,
                                      int64_t N, float eps) {
  FFK_REQUIRE(M >= 0 && N > 0 && N < (1ll << 31), "layer_norm_forward: bad shape");
  if (M == 0) return FFK_OK;
  FFK_REQUIRE(M < (1ll << 31), "layer_norm_forward: too many rows");
  FFK_REQUIRE(input && output && mean && rstd, "layer_norm_forward: NULL tensor");
  if (dtype == FFK_FLOAT)
    return ln_forward<float>(as_stream(stream), input, output, gamma, beta, mean, rstd, M, N, eps);
  if (dtype == FFK_BF16)
    return ln_forward<bf16>(as_stream(stream), input, output, gamma, beta, mean, rstd, M, N, eps);
  return fail(FFK_ERR_UNSUPPORTED, "layer_norm_forward: dtype %d not supported", dtype);
}

extern "C" size_t ffk_layer_norm_backward_workspace_bytes(int64_t M, int64_t N) {
  int64_t blocks = M < kLnBwdMaxBlocks ? M : kLnBwdMaxBlocks;
  if (blocks < 1) blocks = 1;
  return (size_t)blocks * 2 * (size_t)N * sizeof(float);
}

extern "C" int ffk_layer_norm_backward(
    ffk_stream_t stream, int dtype, void const *output_grad, void const *input,
    float const *mean, float const *rstd, void const *gamma, void *input_grad,
    void *gamma_grad, void *beta_grad, int64_t M, int64_t N, void *workspace,
    size_t workspace_bytes, int accumulate_input_grad) {
  FFK_REQUIRE(M >= 0 && N > 0 && N < (1ll << 31), "layer_norm_backward: bad shape");
  if (M == 0) return FFK_OK;
  FFK_REQUIRE(M < (1ll << 31), "layer_norm_backward: too many rows");
  FFK_REQUIRE(output_grad && input && mean && rstd, "layer_norm_backward: NULL tensor");
  FFK_REQUIRE((accumulate_input_grad & ~(FFK_LN_ACC_INPUT | FFK_LN_ACC_PARAMS)) == 0,
              "layer_norm_backward: accumulate_input_grad %d is not a mask of FFK_LN_ACC_INPUT | FFK_LN_ACC_PARAMS",
              accumulate_input_grad);
  bool const acc = (accumulate_input_grad & FFK_LN_ACC_INPUT) != 0;
  bool const acc_params = (accumulate_input_grad & FFK_LN_ACC_PARAMS) != 0;
  if (dtype == FFK_FLOAT)
    return ln_backward<float>(as_stream(stream), output_grad, input, mean, rstd, gamma,
                              input_grad, gamma_grad, beta_grad, M, N, workspace,
                              workspace_bytes, acc, nullptr, nullptr, nullptr, false, acc_params);
  if (dtype == FFK_BF16)
    return ln_backward<bf16>(as_stream(stream), output_grad, input, mean, rstd, gamma,
                             input_grad, gamma_grad, beta_grad, M, N, workspace,
                             workspace_bytes, acc, nullptr, nullptr, nullptr, false, acc_params);
  return fail(FFK_ERR_UNSUPPORTED, "layer_norm_backward: dtype %d not supported", dtype);
}

extern "C" int ffk_layer_norm_backward_residual(
    ffk_stream_t stream, int dtype, void const *output_grad, void const *input, float const *mean,
    float const *rstd, void const *gamma, void const *residual, void *input_grad, void *gamma_grad,
    void *beta_grad, int64_t M, int64_t N, void *workspace, size_t workspace_bytes, int accumulate_params,
    void *dropped_grad, float rate, uint64_t seed, uint64_t offset) {
  FFK_REQUIRE(M >= 0 && N > 0 && N < (1ll << 31), "layer_norm_backward_residual: bad shape");
  if (M == 0) return FFK_OK;
  FFK_REQUIRE(M < (1ll << 31), "layer_norm_backward_residual: too many rows");
  FFK_REQUIRE(output_grad && input && mean && rstd && residual && input_grad,
              "layer_norm_backward_residual: NULL tensor");
  if (dtype != FFK_FLOAT && dtype != FFK_BF16)
    return fail(FFK_ERR_UNSUPPORTED, "layer_norm_backward_residual: dtype %d not supported", dtype);
  return layer_norm_backward_add_residual(as_stream(stream), dtype, output_grad, input, mean, rstd, gamma, residual,
                                          input_grad, gamma_grad, beta_grad, M, N, workspace, workspace_bytes,
                                          dropped_grad, rate, seed, offset, accumulate_params != 0, false);
}

extern "C" int ffk_dropout_add_layer_norm_forward(ffk_stream_t stream, int dtype, void const *input,
                                                  void const *residual, void *sum, void *output, void const *gamma,
                                                  void const *beta, float *mean, float *rstd, int64_t M, int64_t N,
                                                  float eps, float rate, uint64_t seed, uint64_t offset) {
  FFK_REQUIRE(M >= 0 && N > 0, "dropout_add_layer_norm_forward: bad shape");
  if (M == 0) return FFK_OK;
  return dropout_add_layer_norm_forward(as_stream(stream), dtype, input, residual, sum, output, gamma, beta, mean,
                                        rstd, M, N, eps, rate, seed, offset);
}

// ---- the entry point that allocates nothing ---------------------------------
// The per-workgroup partial sums of the parameter gradients, which
// ffk_layer_norm_backward takes from its caller's workspace, live in this
// array instead.  Every device the library runs on holds its own copy at its
// own address until the process ends; host code only ever uses the address
// that hipGetSymbolAddress returned for the device that was current.
constexpr size_t kStaticScratchBytes = FFK_LAYER_NORM_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) float scratch[kStaticScratchBytes / sizeof(float)];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
float *g_scratch_ptr[kMaxDevices];  // per device, filled on that device's first call

int static_scratch_for_current_device(float **out) {
  int dev = -1;
  FFK_HIP(hipGetDevice(&dev));
  FFK_REQUIRE(dev >= 0 && dev < kMaxDevices, "layer_norm_backward_static: device ordinal %d out of range", dev);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    float *p = nullptr;
    FFK_HIP(hipGetSymbolAddress((void **)&p, HIP_SYMBOL(scratch)));
    FFK_REQUIRE(p != nullptr, "layer_norm_backward_static: no device address for the scratch array");
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return FFK_OK;
}
}  // namespace

extern "C" int ffk_layer_norm_backward_static(
    ffk_stream_t stream, int dtype, void const *output_grad, void const *input,
    float const *mean, float const *rstd, void const *gamma, void *input_grad,
    void *gamma_grad, void *beta_grad, int64_t M, int64_t N,
    int accumulate_input_grad) {
  FFK_REQUIRE(M >= 0 && N > 0 && N < (1ll << 31), "layer_norm_backward_static: bad shape");
  if (M == 0) return FFK_OK;
  FFK_REQUIRE(M < (1ll << 31), "layer_norm_backward_static: too many rows");
  FFK_REQUIRE(output_grad && input && mean && rstd, "layer_norm_backward_static: NULL tensor");
  FFK_REQUIRE(dtype == FFK_FLOAT || dtype == FFK_BF16, "layer_norm_backward_static: dtype %d not supported", dtype);
  FFK_REQUIRE((accumulate_input_grad & ~(FFK_LN_ACC_INPUT | FFK_LN_ACC_PARAMS)) == 0,
              "layer_norm_backward_static: accumulate_input_grad %d is not a mask of FFK_LN_ACC_INPUT | "
              "FFK_LN_ACC_PARAMS", accumulate_input_grad);
  if (N > FFK_LAYER_NORM_STATIC_MAX_N) {
    return fail(FFK_ERR_WORKSPACE,
                "layer_norm_backward_static: rows of %lld elements exceed the limit of %d "
                "(the scratch array is %zu bytes per device); use ffk_layer_norm_backward with a workspace",
                (long long)N, FFK_LAYER_NORM_STATIC_MAX_N, kStaticScratchBytes);
  }
  float *ptr = nullptr;
  int rc = static_scratch_for_current_device(&ptr);
  if (rc != FFK_OK) return rc;
  // The array is shared by every call on this device, so its column reduction
  // runs here and now: a collected one would read the partial sums after a
  // later call has overwritten them.
  // A reduction collected earlier on this thread that writes the same
  // gamma_grad / beta_grad (shared LayerNorm parameters) has to reach them
  // first, as the calls were made: run what is collected before this one.
  ColreduceBatch *const collecting = tl_colreduce_batch;
  if (collecting != nullptr) {
    for (int k = 0; k < collecting->count; k++) {
      ColreduceJob const &c = collecting->job[k];
      bool const clash = (gamma_grad != nullptr && (c.out0 == gamma_grad || c.out1 == gamma_grad)) ||
                         (beta_grad != nullptr && (c.out0 == beta_grad || c.out1 == beta_grad));
      if (clash) {
        FFK_HIP(colreduce_flush(as_stream(stream), *collecting));
        break;
      }
    }
  }
  tl_colreduce_batch = nullptr;
  bool const acc = (accumulate_input_grad & FFK_LN_ACC_INPUT) != 0;
  bool const acc_params = (accumulate_input_grad & FFK_LN_ACC_PARAMS) != 0;
  if (dtype == FFK_FLOAT) {
    rc = ln_backward<float>(as_stream(stream), output_grad, input, mean, rstd, gamma, input_grad, gamma_grad,
                            beta_grad, M, N, ptr, kStaticScratchBytes, acc, nullptr, nullptr, nullptr, true, acc_params);
  } else {
    rc = ln_backward<bf16>(as_stream(stream), output_grad, input, mean, rstd, gamma, input_grad, gamma_grad,
                           beta_grad, M, N, ptr, kStaticScratchBytes, acc, nullptr, nullptr, nullptr, true, acc_params);
  }
  tl_colreduce_batch = collecting;
  return rc;
}
