// Fused (flash-style) attention for gfx950 in fp32: the core behind the
// reference's own MultiHeadAttention signature, which hands float tensors to
// cudnnMultiHeadAttnForward / BackwardData (lib/kernels/src/cuda/ops/
// attention_kernels.cu:224,261).  Same scheme as the bf16 core in
// attention.hip -- scores never leave the CU, a lane owns one query row of the
// transposed score tile, the backward is two kernels without atomics -- on the
// fp32 matrix instruction v_mfma_f32_32x32x2f32:
//   A operand: lane l holds A[row l%32][k = l/32]
//   B operand: lane l holds B[k = l/32][column l%32]
//   accumulator element r of lane l: row 8*(r/4) + 4*(l/32) + r%4, column l%32.
// A contraction over the head dim takes DP/2 steps; the lanes of half h = l/32
// walk d = h*DP/2 + step, so both halves read contiguous floats (16-byte LDS
// reads, four steps each).  A contraction over keys or queries re-uses an
// accumulator tile as an operand: step r takes element r of every lane, whose
// reduction index is 8*(r/4) + 4*h + r%4, and the other operand is read from
// the LDS tile row of that index.
// head sizes: any multiple of 4 up to 256, and the value head size (V, O, dO,
// dV) may differ from the query/key one (Q, K, dQ, dK): the reference's model
// builders ask for kdim = vdim = 256 (lib/models/src/models/transformer/
// transformer.cc:37-38, bert/bert.cc:64-65) and the projection sizes are free
// (lib/op-attrs/src/op-attrs/ops/attention.cc:23-37).  DP is the larger of
// the two rounded up to 32, 64, 128 or 256; the missing columns of either
// kind are read as zeros.  At DP = 256 a wave's operands and accumulators no
// longer fit its 512 registers in one pass: tiles are then loaded without a
// register prefetch and dK and dV are produced by two launches of the dK/dV
// kernel (WHAT = 1: dV only, needs K; WHAT = 2: dK only, needs K and V).
#include "ffk_common.h"

namespace ffk {

constexpr float kLog2eF = 1.4426950408889634f;
constexpr float kLn2F = 0.6931471805599453f;

struct AttnF32Params {
  float const *q, *k, *v, *o, *d_o;
  float *out;  // forward: O
  float *lse;  // forward: written; backward: read
  float *delta;
  float *dq, *dk, *dv;
  int B, H, Sq, Skv, Dq, Dv;  // Dq: head size of Q, K, dQ, dK; Dv: of V, O, dO, dV
  int64_t q_bs, q_ss, k_bs, k_ss, v_bs, v_ss, o_bs, o_ss;
  float scale, scale_log2;
  int causal;
};

template <int DP>
struct AttnF32Cfg {
  static constexpr int kBlk = 128;        // rows a workgroup owns
  static constexpr int kTile = 32;        // rows of the streamed operands per step
  static constexpr int kStrideA = DP + 4; // tile read along d only (16-byte reads, conflict-free)
  static constexpr int kStrideB = DP + 8; // tile also read one row per half-wave: 4 rows apart = 32 banks apart
  static constexpr int kChunks = kTile * DP / 4 / 256;  // 16-byte chunks per thread
  static_assert(kTile * DP / 4 % 256 == 0, "tile chunks");
  // next tile fetched into registers while this one is computed on (not at DP = 256: no room)
  static constexpr bool kPrefetch = DP <= 128;
};

__device__ __forceinline__ f32x4 load4_or_zero(float const *row, int d0, int D) {
  f32x4 z = {0.0f, 0.0f, 0.0f, 0.0f};
  return d0 < D ? *reinterpret_cast<f32x4 const *>(row + d0) : z;
}

// This lane's row of an owned operand, in the step order of the d contraction.
template <int DP>
__device__ __forceinline__ void load_owned_row(float const *row, int D, int h32, float (&f)[DP / 2]) {
#pragma unroll
  for (int c = 0; c < DP / 8; c++) {
    f32x4 x = load4_or_zero(row, h32 * (DP / 2) + 4 * c, D);
    f[4 * c] = x[0];
    f[4 * c + 1] = x[1];
    f[4 * c + 2] = x[2];
    f[4 * c + 3] = x[3];
  }
}

// Streamed tile: global -> registers, registers -> LDS.
template <int DP>
__device__ __forceinline__ void tile_gload(float const *base, int64_t row_stride, int row0, int last_row, int D,
                                           int t, f32x4 (&r)[AttnF32Cfg<DP>::kChunks]) {
#pragma unroll
  for (int i = 0; i < AttnF32Cfg<DP>::kChunks; i++) {
    int const c = t + i * 256;
    int const row = c / (DP / 4), ch = c % (DP / 4);
    int const gr = min(row0 + row, last_row);
    r[i] = load4_or_zero(base + (int64_t)gr * row_stride, ch * 4, D);
  }
}
template <int DP, int STRIDE>
__device__ __forceinline__ void tile_lstore(float *tile, int t, f32x4 const (&r)[AttnF32Cfg<DP>::kChunks]) {
#pragma unroll
  for (int i = 0; i < AttnF32Cfg<DP>::kChunks; i++) {
    int const c = t + i * 256;
    int const row = c / (DP / 4), ch = c % (DP / 4);
    *reinterpret_cast<f32x4 *>(tile + row * STRIDE + ch * 4) = r[i];
  }
}

// acc (+)= T . owned^T over d: rows = the tile's rows, columns = the owned rows
// of this wave (one per lane and half).  tile_lane = tile + (l%32)*stride + h*DP/2.
template <int DP>
__device__ __forceinline__ void contract_d(float const *tile_lane, float const (&owned)[DP / 2], f32x16 &acc) {
#pragma unroll
  for (int c = 0; c < DP / 8; c++) {
    f32x4 const a = *reinterpret_cast<f32x4 const *>(tile_lane + 4 * c);
#pragma unroll
    for (int e = 0; e < 4; e++) {
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[e], owned[4 * c + e], acc, 0, 0, 0);
    }
  }
}

// --------------------------------------------------------------------------
// forward: workgroup = 128 query rows of one (batch, head), 32 per wave
// --------------------------------------------------------------------------
template <int DP>
__global__ __launch_bounds__(256) void attn_f32_fwd_kernel(AttnF32Params p) {
  using C = AttnF32Cfg<DP>;
  __shared__ __attribute__((aligned(16))) float Ks[2][C::kTile * C::kStrideA];
  __shared__ __attribute__((aligned(16))) float Vs[2][C::kTile * C::kStrideB];
  int const t = threadIdx.x, lane = t & 63, h32 = lane >> 5, l32 = lane & 31;
  int const wave = __builtin_amdgcn_readfirstlane(t >> 6);
  int const nqb = (p.Sq + C::kBlk - 1) / C::kBlk;
  int const hb = blockIdx.x % (p.H * p.B);
  int const qb = nqb - 1 - blockIdx.x / (p.H * p.B);  // heaviest causal blocks first
  int const head = hb % p.H, b = hb / p.H;
  int const q0 = qb * C::kBlk;
  int const qrow = q0 + wave * 32 + l32;
  float const *qp = p.q + (int64_t)b * p.q_bs + (int64_t)head * p.Dq;
  float const *kp = p.k + (int64_t)b * p.k_bs + (int64_t)head * p.Dq;
  float const *vp = p.v + (int64_t)b * p.v_bs + (int64_t)head * p.Dv;

  float qf[DP / 2];
  load_owned_row<DP>(qp + (int64_t)min(qrow, p.Sq - 1) * p.q_ss, p.Dq, h32, qf);

  int kv_end = p.Skv;
  if (p.causal) kv_end = min(p.Skv, q0 + C::kBlk);
  int const ntiles = (kv_end + C::kTile - 1) / C::kTile;

  f32x16 oacc[DP / 32];
#pragma unroll
  for (int i = 0; i < DP / 32; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) oacc[i][r] = 0.0f;
  float m_run = -INFINITY, l_run = 0.0f;

  f32x4 rk[C::kChunks], rv[C::kChunks];
  auto fetch = [&](int kv0) {
    tile_gload<DP>(kp, p.k_ss, kv0, p.Skv - 1, p.Dq, t, rk);
    tile_gload<DP>(vp, p.v_ss, kv0, p.Skv - 1, p.Dv, t, rv);
  };
  auto stash = [&](int buf) {
    tile_lstore<DP, C::kStrideA>(Ks[buf], t, rk);
    tile_lstore<DP, C::kStrideB>(Vs[buf], t, rv);
  };
  fetch(0);
  stash(0);
  __syncthreads();
  int cur = 0;
  for (int it = 0; it < ntiles; it++) {
    int const kv0 = it * C::kTile;
    bool const more = it + 1 < ntiles;
    if (C::kPrefetch && more) fetch(kv0 + C::kTile);
    // a wave whose rows all lie before this tile (causal) has nothing to add
    bool const active = !p.causal || kv0 <= q0 + wave * 32 + 31;
    if (active) {
      // S^T: rows = keys of the tile, column = this lane's query
      f32x16 s;
#pragma unroll
      for (int r = 0; r < 16; r++) s[r] = 0.0f;
      contract_d<DP>(Ks[cur] + l32 * C::kStrideA + h32 * (DP / 2), qf, s);
      bool const need_mask = (kv0 + C::kTile > p.Skv) || (p.causal && kv0 + C::kTile - 1 > q0 + wave * 32);
      if (need_mask) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
          int const kv = kv0 + 8 * (r >> 2) + 4 * h32 + (r & 3);
          if (kv >= p.Skv || (p.causal && kv > qrow)) s[r] = -INFINITY;
        }
      }
      float mx = -INFINITY;
#pragma unroll
      for (int r = 0; r < 16; r++) mx = fmaxf(mx, s[r]);
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64)) * p.scale_log2;
      // finite from the first tile on: key 0 is visible to every query
      float const m_new = fmaxf(m_run, mx);
      float const alpha = __builtin_amdgcn_exp2f(m_run - m_new);
      float sum = 0.0f;
      float pv[16];
#pragma unroll
      for (int r = 0; r < 16; r++) {
        pv[r] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[r], p.scale_log2, -m_new));
        sum += pv[r];
      }
      sum += __shfl_xor(sum, 32, 64);
      l_run = l_run * alpha + sum;
      m_run = m_new;
      if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
        for (int i = 0; i < DP / 32; i++)
#pragma unroll
          for (int r = 0; r < 16; r++) oacc[i][r] *= alpha;
      }
      // O^T += V^T P^T: A = V^T (row d), B = P^T (column = query), reduction over keys
      float const *vt = Vs[cur] + (4 * h32) * C::kStrideB + l32;
#pragma unroll
      for (int r = 0; r < 16; r++) {
        int const krow = 8 * (r >> 2) + (r & 3);
#pragma unroll
        for (int i = 0; i < DP / 32; i++) {
          oacc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(vt[krow * C::kStrideB + i * 32], pv[r], oacc[i], 0, 0, 0);
        }
      }
    }
    if (more) {
      if (!C::kPrefetch) fetch(kv0 + C::kTile);
      stash(cur ^ 1);
    }
    __syncthreads();
    cur ^= 1;
  }

  if (qrow < p.Sq) {
    float const inv = 1.0f / l_run;
    float *op = p.out + (int64_t)b * p.o_bs + (int64_t)qrow * p.o_ss + (int64_t)head * p.Dv;
#pragma unroll
    for (int i = 0; i < DP / 32; i++) {
#pragma unroll
      for (int g = 0; g < 4; g++) {
        int const d = i * 32 + 8 * g + 4 * h32;
        if (d < p.Dv) {
          f32x4 w = {oacc[i][4 * g] * inv, oacc[i][4 * g + 1] * inv, oacc[i][4 * g + 2] * inv,
                     oacc[i][4 * g + 3] * inv};
          *reinterpret_cast<f32x4 *>(op + d) = w;
        }
      }
    }
    if (h32 == 0 && p.lse != nullptr) {
      p.lse[((int64_t)b * p.H + head) * p.Sq + qrow] = (m_run + __log2f(l_run)) * kLn2F;
    }
  }
}

// delta[b,h,q] = sum_d O * dO; DP/4 lanes share a row
template <int DP>
__global__ __launch_bounds__(256) void attn_f32_delta_kernel(AttnF32Params p) {
  constexpr int LPR = DP / 4;
  constexpr int RPW = 64 / LPR;
  int const lane = threadIdx.x & 63;
  int64_t const row = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * RPW + lane / LPR;
  int64_t const total = (int64_t)p.B * p.H * p.Sq;
  float s = 0.0f;
  bool const ok = row < total;
  int head = 0, q = 0, b = 0;
  if (ok) {
    head = (int)(row % p.H);
    q = (int)((row / p.H) % p.Sq);
    b = (int)(row / ((int64_t)p.Sq * p.H));
    int64_t const off = (int64_t)b * p.o_bs + (int64_t)q * p.o_ss + (int64_t)head * p.Dv;
    int const d0 = (lane % LPR) * 4;
    f32x4 const o = load4_or_zero(p.o + off, d0, p.Dv);
    f32x4 const g = load4_or_zero(p.d_o + off, d0, p.Dv);
    s = o[0] * g[0] + o[1] * g[1] + o[2] * g[2] + o[3] * g[3];
  }
#pragma unroll
  for (int m = 1; m < LPR; m <<= 1) s += __shfl_xor(s, m, 64);
  if (ok && lane % LPR == 0) p.delta[((int64_t)b * p.H + head) * p.Sq + q] = s;
}

// --------------------------------------------------------------------------
// backward (A): dK, dV.  Workgroup owns 128 key rows, streams query tiles.
// WHAT: bit 0 = produce dV, bit 1 = produce dK.
// --------------------------------------------------------------------------
template <int DP, int WHAT>
__global__ __launch_bounds__(256) void attn_f32_bwd_dkdv_kernel(AttnF32Params p) {
  using C = AttnF32Cfg<DP>;
  constexpr bool kDV = (WHAT & 1) != 0, kDK = (WHAT & 2) != 0;
  // dV needs the dO tile as an operand, dK needs it for dP: both
  __shared__ __attribute__((aligned(16))) float Qs[2][C::kTile * C::kStrideB];
  __shared__ __attribute__((aligned(16))) float Gs[2][C::kTile * C::kStrideB];  // dO
  __shared__ __attribute__((aligned(16))) float Ls[2][C::kTile], Ds[2][C::kTile];
  int const t = threadIdx.x, lane = t & 63, h32 = lane >> 5, l32 = lane & 31;
  int const wave = __builtin_amdgcn_readfirstlane(t >> 6);
  int const hb = blockIdx.x % (p.H * p.B);
  int const head = hb % p.H, b = hb / p.H;
  int const kv0 = (blockIdx.x / (p.H * p.B)) * C::kBlk;
  int const kvrow = kv0 + wave * 32 + l32;
  float const *qp = p.q + (int64_t)b * p.q_bs + (int64_t)head * p.Dq;
  float const *gp = p.d_o + (int64_t)b * p.o_bs + (int64_t)head * p.Dv;
  float const *kp = p.k + (int64_t)b * p.k_bs + (int64_t)head * p.Dq;
  float const *vp = p.v + (int64_t)b * p.v_bs + (int64_t)head * p.Dv;
  float const *lsep = p.lse + ((int64_t)b * p.H + head) * p.Sq;
  float const *delp = p.delta + ((int64_t)b * p.H + head) * p.Sq;

  float kf[DP / 2];
  float vf[kDK ? DP / 2 : 1];
  load_owned_row<DP>(kp + (int64_t)min(kvrow, p.Skv - 1) * p.k_ss, p.Dq, h32, kf);
  if constexpr (kDK) load_owned_row<DP>(vp + (int64_t)min(kvrow, p.Skv - 1) * p.v_ss, p.Dv, h32, vf);
  f32x16 dk[kDK ? DP / 32 : 1], dv[kDV ? DP / 32 : 1];
#pragma unroll
  for (int i = 0; i < (kDK ? DP / 32 : 1); i++)
#pragma unroll
    for (int r = 0; r < 16; r++) dk[i][r] = 0.0f;
#pragma unroll
  for (int i = 0; i < (kDV ? DP / 32 : 1); i++)
#pragma unroll
    for (int r = 0; r < 16; r++) dv[i][r] = 0.0f;

  int const q_begin = p.causal ? (kv0 / C::kTile) * C::kTile : 0;
  int const ntiles = q_begin < p.Sq ? (p.Sq - q_begin + C::kTile - 1) / C::kTile : 0;

  f32x4 rq[C::kChunks], rg[C::kChunks];
  float rl = 0.0f, rd = 0.0f;
  auto gload = [&](int qt0) {
    tile_gload<DP>(qp, p.q_ss, qt0, p.Sq - 1, p.Dq, t, rq);
    tile_gload<DP>(gp, p.o_ss, qt0, p.Sq - 1, p.Dv, t, rg);
    int const gr = min(qt0 + (t & (C::kTile - 1)), p.Sq - 1);
    rl = lsep[gr] * kLog2eF;
    rd = delp[gr];
  };
  auto lstore = [&](int buf) {
    tile_lstore<DP, C::kStrideB>(Qs[buf], t, rq);
    tile_lstore<DP, C::kStrideB>(Gs[buf], t, rg);
    if (t < C::kTile) {
      Ls[buf][t] = rl;
      Ds[buf][t] = rd * p.scale;
    }
  };
  if (ntiles > 0) {
    gload(q_begin);
    lstore(0);
  }
  __syncthreads();
  int cur = 0;
  for (int it = 0; it < ntiles; it++) {
    int const qt0 = q_begin + it * C::kTile;
    bool const more = it + 1 < ntiles;
    if (C::kPrefetch && more) gload(qt0 + C::kTile);
    // a wave whose keys all lie after this query tile (causal) contributes nothing
    bool const active = !p.causal || kv0 + wave * 32 <= qt0 + C::kTile - 1;
    if (active) {
      // S = Q K^T, dP = dO V^T: rows = queries of the tile, column = this lane's key
      f32x16 s, dp;
#pragma unroll
      for (int r = 0; r < 16; r++) {
        s[r] = 0.0f;
        dp[r] = 0.0f;
      }
      contract_d<DP>(Qs[cur] + l32 * C::kStrideB + h32 * (DP / 2), kf, s);
      if constexpr (kDK) contract_d<DP>(Gs[cur] + l32 * C::kStrideB + h32 * (DP / 2), vf, dp);
      float pv[16], dsv[16];
#pragma unroll
      for (int r = 0; r < 16; r++) {
        int const ql = 8 * (r >> 2) + 4 * h32 + (r & 3);
        int const qg = qt0 + ql;
        float const e = __builtin_amdgcn_exp2f(__builtin_fmaf(s[r], p.scale_log2, -Ls[cur][ql]));
        bool const masked = qg >= p.Sq || kvrow >= p.Skv || (p.causal && kvrow > qg);
        pv[r] = masked ? 0.0f : e;
        // dS = P (dP - delta) scale; Ds holds delta * scale
        dsv[r] = masked ? 0.0f : e * __builtin_fmaf(dp[r], p.scale, -Ds[cur][ql]);
      }
      // dV += P^T dO, dK += dS^T Q: A = the accumulator (row = key), B = dO / Q rows of the
      // matching query, reduction over the tile's queries
      float const *gt = Gs[cur] + (4 * h32) * C::kStrideB + l32;
      float const *qt = Qs[cur] + (4 * h32) * C::kStrideB + l32;
#pragma unroll
      for (int r = 0; r < 16; r++) {
        int const qr = 8 * (r >> 2) + (r & 3);
#pragma unroll
        for (int i = 0; i < DP / 32; i++) {
          if constexpr (kDV) {
            dv[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(pv[r], gt[qr * C::kStrideB + i * 32], dv[i], 0, 0, 0);
          }
          if constexpr (kDK) {
            dk[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(dsv[r], qt[qr * C::kStrideB + i * 32], dk[i], 0, 0, 0);
          }
        }
      }
    }
    if (more) {
      if (!C::kPrefetch) gload(qt0 + C::kTile);
      lstore(cur ^ 1);
    }
    __syncthreads();
    cur ^= 1;
  }

  // accumulator element r: key row 8*(r/4) + 4*h + r%4 of this wave's 32, column d = i*32 + l%32:
  // the 32 lanes of a half write 128 contiguous bytes of one row
  float *dkp = p.dk + (int64_t)b * p.k_bs + (int64_t)head * p.Dq;
  float *dvp = p.dv + (int64_t)b * p.v_bs + (int64_t)head * p.Dv;
#pragma unroll
  for (int i = 0; i < DP / 32; i++) {
    int const d = i * 32 + l32;
#pragma unroll
    for (int r = 0; r < 16; r++) {
      int const grow = kv0 + wave * 32 + 8 * (r >> 2) + 4 * h32 + (r & 3);
      if (grow < p.Skv) {
        if constexpr (kDK) {
          if (d < p.Dq) dkp[(int64_t)grow * p.k_ss + d] = dk[i][r];
        }
        if constexpr (kDV) {
          if (d < p.Dv) dvp[(int64_t)grow * p.v_ss + d] = dv[i][r];
        }
      }
    }
  }
}

// --------------------------------------------------------------------------
// backward (B): dQ.  Workgroup owns 128 query rows, streams key tiles.
// --------------------------------------------------------------------------
template <int DP>
__global__ __launch_bounds__(256) void attn_f32_bwd_dq_kernel(AttnF32Params p) {
  using C = AttnF32Cfg<DP>;
  __shared__ __attribute__((aligned(16))) float Ks[2][C::kTile * C::kStrideB];
  __shared__ __attribute__((aligned(16))) float Vs[2][C::kTile * C::kStrideA];
  int const t = threadIdx.x, lane = t & 63, h32 = lane >> 5, l32 = lane & 31;
  int const wave = __builtin_amdgcn_readfirstlane(t >> 6);
  int const nqb = (p.Sq + C::kBlk - 1) / C::kBlk;
  int const hb = blockIdx.x % (p.H * p.B);
  int const qb = nqb - 1 - blockIdx.x / (p.H * p.B);
  int const head = hb % p.H, b = hb / p.H;
  int const q0 = qb * C::kBlk;
  int const qrow = q0 + wave * 32 + l32;
  float const *qp = p.q + (int64_t)b * p.q_bs + (int64_t)head * p.Dq;
  float const *gp = p.d_o + (int64_t)b * p.o_bs + (int64_t)head * p.Dv;
  float const *kp = p.k + (int64_t)b * p.k_bs + (int64_t)head * p.Dq;
  float const *vp = p.v + (int64_t)b * p.v_bs + (int64_t)head * p.Dv;

  float qf[DP / 2], gf[DP / 2];
  int const rq = min(qrow, p.Sq - 1);
  load_owned_row<DP>(qp + (int64_t)rq * p.q_ss, p.Dq, h32, qf);
  load_owned_row<DP>(gp + (int64_t)rq * p.o_ss, p.Dv, h32, gf);
  float const lse2 = p.lse[((int64_t)b * p.H + head) * p.Sq + rq] * kLog2eF;
  float const delta_s = p.delta[((int64_t)b * p.H + head) * p.Sq + rq] * p.scale;
  f32x16 dq[DP / 32];
#pragma unroll
  for (int i = 0; i < DP / 32; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) dq[i][r] = 0.0f;

  int kv_end = p.Skv;
  if (p.causal) kv_end = min(p.Skv, q0 + C::kBlk);
  int const ntiles = (kv_end + C::kTile - 1) / C::kTile;

  f32x4 rk[C::kChunks], rv[C::kChunks];
  auto fetch = [&](int kt0) {
    tile_gload<DP>(kp, p.k_ss, kt0, p.Skv - 1, p.Dq, t, rk);
    tile_gload<DP>(vp, p.v_ss, kt0, p.Skv - 1, p.Dv, t, rv);
  };
  auto stash = [&](int buf) {
    tile_lstore<DP, C::kStrideB>(Ks[buf], t, rk);
    tile_lstore<DP, C::kStrideA>(Vs[buf], t, rv);
  };
  fetch(0);
  stash(0);
  __syncthreads();
  int cur = 0;
  for (int it = 0; it < ntiles; it++) {
    int const kt0 = it * C::kTile;
    bool const more = it + 1 < ntiles;
    if (C::kPrefetch && more) fetch(kt0 + C::kTile);
    bool const active = !p.causal || kt0 <= q0 + wave * 32 + 31;
    if (active) {
      // S^T = K Q^T, dP^T = V dO^T: rows = keys of the tile, column = this lane's query
      f32x16 s, dp;
#pragma unroll
      for (int r = 0; r < 16; r++) {
        s[r] = 0.0f;
        dp[r] = 0.0f;
      }
      contract_d<DP>(Ks[cur] + l32 * C::kStrideB + h32 * (DP / 2), qf, s);
      contract_d<DP>(Vs[cur] + l32 * C::kStrideA + h32 * (DP / 2), gf, dp);
      float dsv[16];
#pragma unroll
      for (int r = 0; r < 16; r++) {
        int const kv = kt0 + 8 * (r >> 2) + 4 * h32 + (r & 3);
        float const e = __builtin_amdgcn_exp2f(__builtin_fmaf(s[r], p.scale_log2, -lse2));
        bool const masked = kv >= p.Skv || (p.causal && kv > qrow);
        dsv[r] = masked ? 0.0f : e * __builtin_fmaf(dp[r], p.scale, -delta_s);
      }
      // dQ^T += K^T dS^T: A = K^T (row d), B = dS^T, reduction over the tile's keys
      float const *kt = Ks[cur] + (4 * h32) * C::kStrideB + l32;
#pragma unroll
      for (int r = 0; r < 16; r++) {
        int const krow = 8 * (r >> 2) + (r & 3);
#pragma unroll
        for (int i = 0; i < DP / 32; i++) {
          dq[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(kt[krow * C::kStrideB + i * 32], dsv[r], dq[i], 0, 0, 0);
        }
      }
    }
    if (more) {
      if (!C::kPrefetch) fetch(kt0 + C::kTile);
      stash(cur ^ 1);
    }
    __syncthreads();
    cur ^= 1;
  }

  if (qrow < p.Sq) {
    float *dqp = p.dq + (int64_t)b * p.q_bs + (int64_t)qrow * p.q_ss + (int64_t)head * p.Dq;
#pragma unroll
    for (int i = 0; i < DP / 32; i++) {
#pragma unroll
      for (int g = 0; g < 4; g++) {
        int const d = i * 32 + 8 * g + 4 * h32;
        if (d < p.Dq) {
          f32x4 w = {dq[i][4 * g], dq[i][4 * g + 1], dq[i][4 * g + 2], dq[i][4 * g + 3]};
          *reinterpret_cast<f32x4 *>(dqp + d) = w;
        }
      }
    }
  }
}

static int check_desc_f32(char const *who, ffk_attention_desc_t const *d) {
  int64_t const dq = d->head_dim, dv = d->v_head_dim > 0 ? d->v_head_dim : d->head_dim;
  FFK_REQUIRE(dq > 0 && dq <= 256 && dq % 4 == 0 && dv <= 256 && dv % 4 == 0,
              "%s: fp32 head_dim %lld / v_head_dim %lld not supported (multiples of 4 up to 256)", who,
              (long long)dq, (long long)dv);
  FFK_REQUIRE(d->batch > 0 && d->heads > 0 && d->seq_q > 0 && d->seq_kv > 0, "%s: bad shape", who);
  FFK_REQUIRE(d->batch * d->heads * ((d->seq_q > d->seq_kv ? d->seq_q : d->seq_kv) / 128 + 1) < (1ll << 31),
              "%s: too many workgroups", who);
  FFK_REQUIRE(d->seq_q < (1ll << 30) && d->seq_kv < (1ll << 30), "%s: sequence too long", who);
  FFK_REQUIRE(d->q_seq_stride % 4 == 0 && d->k_seq_stride % 4 == 0 && d->v_seq_stride % 4 == 0 &&
                  d->o_seq_stride % 4 == 0 && d->q_batch_stride % 4 == 0 && d->k_batch_stride % 4 == 0 &&
                  d->v_batch_stride % 4 == 0 && d->o_batch_stride % 4 == 0,
              "%s: fp32 strides must be multiples of 4 elements", who);
  FFK_REQUIRE(d->q_seq_stride >= d->heads * dq && d->k_seq_stride >= d->heads * dq &&
                  d->v_seq_stride >= d->heads * dv && d->o_seq_stride >= d->heads * dv,
              "%s: sequence stride smaller than heads * head_dim", who);
  return FFK_OK;
}

static AttnF32Params make_params(ffk_attention_desc_t const *d) {
  AttnF32Params p = {};
  p.B = (int)d->batch; p.H = (int)d->heads; p.Sq = (int)d->seq_q; p.Skv = (int)d->seq_kv;
  p.Dq = (int)d->head_dim;
  p.Dv = (int)(d->v_head_dim > 0 ? d->v_head_dim : d->head_dim);
  p.q_bs = d->q_batch_stride; p.q_ss = d->q_seq_stride;
  p.k_bs = d->k_batch_stride; p.k_ss = d->k_seq_stride;
  p.v_bs = d->v_batch_stride; p.v_ss = d->v_seq_stride;
  p.o_bs = d->o_batch_stride; p.o_ss = d->o_seq_stride;
  p.scale = d->scale;
  p.scale_log2 = d->scale * kLog2eF;
  p.causal = d->causal;
  return p;
}

#define FFK_ATTN_F32_DISPATCH(D_, CALL)                                        \
  do {                                                                         \
    if ((D_) <= 32) { CALL(32); }                                              \
    else if ((D_) <= 64) { CALL(64); }                                         \
    else if ((D_) <= 128) { CALL(128); }                                       \
    else { CALL(256); }                                                        \
  } while (0)

int attention_f32_forward(hipStream_t st, ffk_attention_desc_t const *d, void const *q, void const *k,
                          void const *v, void *o, float *lse) {
  int rc = check_desc_f32("attention_forward", d);
  if (rc != FFK_OK) return rc;
  AttnF32Params p = make_params(d);
  p.q = static_cast<float const *>(q);
  p.k = static_cast<float const *>(k);
  p.v = static_cast<float const *>(v);
  p.out = static_cast<float *>(o);
  p.lse = lse;
  unsigned const grid = (unsigned)(ceil_div(p.Sq, 128) * p.H * p.B);
  int const dmax = p.Dq > p.Dv ? p.Dq : p.Dv;
#define CALL(DP_) attn_f32_fwd_kernel<DP_><<<grid, 256, 0, st>>>(p)
  FFK_ATTN_F32_DISPATCH(dmax, CALL);
#undef CALL
  FFK_CHECK_LAUNCH();
  return FFK_OK;
}

template <int DP>
static void launch_f32_backward(hipStream_t st, AttnF32Params const &p, int64_t rows, unsigned gkv, unsigned gq) {
  attn_f32_delta_kernel<DP><<<(unsigned)ceil_div(rows, 4 * (64 / (DP / 4))), 256, 0, st>>>(p);
  if constexpr (DP <= 128) {
    attn_f32_bwd_dkdv_kernel<DP, 3><<<gkv, 256, 0, st>>>(p);
  } else {
    attn_f32_bwd_dkdv_kernel<DP, 1><<<gkv, 256, 0, st>>>(p);
    attn_f32_bwd_dkdv_kernel<DP, 2><<<gkv, 256, 0, st>>>(p);
  }
  attn_f32_bwd_dq_kernel<DP><<<gq, 256, 0, st>>>(p);
}

int attention_f32_backward(hipStream_t st, ffk_attention_desc_t const *d, void const *q, void const *k,
                           void const *v, void const *o, void const *d_o, float const *lse, float *delta,
                           void *dq, void *dk, void *dv) {
  int rc = check_desc_f32("attention_backward", d);
  if (rc != FFK_OK) return rc;
  AttnF32Params p = make_params(d);
  p.q = static_cast<float const *>(q);
  p.k = static_cast<float const *>(k);
  p.v = static_cast<float const *>(v);
  p.o = static_cast<float const *>(o);
  p.d_o = static_cast<float const *>(d_o);
  p.lse = const_cast<float *>(lse);
  p.delta = delta;
  p.dq = static_cast<float *>(dq);
  p.dk = static_cast<float *>(dk);
  p.dv = static_cast<float *>(dv);
  int64_t const rows = (int64_t)p.B * p.H * p.Sq;
  unsigned const gkv = (unsigned)(ceil_div(p.Skv, 128) * p.H * p.B);
  unsigned const gq = (unsigned)(ceil_div(p.Sq, 128) * p.H * p.B);
  int const dmax = p.Dq > p.Dv ? p.Dq : p.Dv;
#define CALL(DP_) launch_f32_backward<DP_>(st, p, rows, gkv, gq)
  FFK_ATTN_F32_DISPATCH(dmax, CALL);
#undef CALL
  FFK_CHECK_LAUNCH();
  return FFK_OK;
}

}  // namespace ffk
