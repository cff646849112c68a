// Fused attention for gfx950, bf16 operands / fp32 accumulation, for the head
// sizes the tuned kernels of attention.hip do not take: any multiple of 8 up to
// 256, and a value head size (V, O, dO, dV) that differs from the query/key one
// (Q, K, dQ, dK).  The reference's model builders ask for kdim = vdim = 256
// (lib/models/src/models/transformer/transformer.cc:37-38, bert/bert.cc:64-65)
// and its attributes leave the two projection sizes free
// (lib/op-attrs/src/op-attrs/ops/attention.cc:23-37).
//
// Same scheme as attention.hip (scores computed transposed so a lane owns one
// query's column, probabilities fed to the next product from registers, the
// backward as two kernels without atomics), written for generality: DP is the
// larger head size rounded up to 64, 128 or 256, columns past a tensor's own
// head size are read as zeros and never stored, tiles are 32 rows and travel
// global -> registers -> LDS one step ahead.  At DP = 256 a wave's operands and
// accumulators do not fit its registers in one pass: tiles are then fetched
// without the register prefetch, and dK and dV come from two launches of the
// dK/dV kernel (WHAT = 1: dV only; WHAT = 2: dK only).
#include "attention_common.h"

namespace ffk {

struct AttnGenParams {
  bf16 const *q, *k, *v, *o, *d_o;
  bf16 *out;
  float *lse;    // forward: written; backward: read
  float *delta;  // backward: written by the dQ kernel, read by the dK/dV kernel
  bf16 *dq, *dk, *dv;
  int B, H, Sq, Skv, Dq, Dv;
  int64_t q_bs, q_ss, k_bs, k_ss, v_bs, v_ss, o_bs, o_ss;
  float scale, scale_log2;
  int causal;
};

template <int DP>
struct AttnGenCfg {
  static constexpr int kBlk = 128;        // rows owned by a workgroup (32 per wave)
  static constexpr int kTile = 32;        // rows of the streamed operands per step
  static constexpr int kStride = DP + 40; // serves the 16-byte row reads and the transposing reads
  static constexpr int kChunks = kTile * DP / 8 / 256;  // 16-byte chunks per thread and tile
  static_assert(kTile * DP / 8 % 256 == 0, "tile chunks");
  static constexpr bool kPrefetch = DP <= 128;
};

__device__ __forceinline__ u32x4 load8_or_zero(bf16 const *row, int d0, int D) {
  u32x4 z = {0u, 0u, 0u, 0u};
  return d0 < D ? *reinterpret_cast<u32x4 const *>(row + d0) : z;
}

// This lane's row of an owned operand as B-operand fragments (column = the row, k = d).
template <int DP>
__device__ __forceinline__ void gen_load_owned(bf16 const *row, int D, int h32, bf16x8 (&f)[DP / 16]) {
#pragma unroll
  for (int kk = 0; kk < DP / 16; kk++) {
    union {
      u32x4 u;
      bf16x8 b;
    } x;
    x.u = load8_or_zero(row, kk * 16 + h32 * 8, D);
    f[kk] = x.b;
  }
}

template <int DP>
__device__ __forceinline__ void gen_tile_gload(bf16 const *base, int64_t row_stride, int row0, int last_row, int D,
                                               int t, u32x4 (&r)[AttnGenCfg<DP>::kChunks]) {
#pragma unroll
  for (int i = 0; i < AttnGenCfg<DP>::kChunks; i++) {
    int const c = t + i * 256;
    int const row = c / (DP / 8), ch = c % (DP / 8);
    int const gr = min(row0 + row, last_row);
    r[i] = load8_or_zero(base + (int64_t)gr * row_stride, ch * 8, D);
  }
}
template <int DP>
__device__ __forceinline__ void gen_tile_lstore(bf16 *tile, int t, u32x4 const (&r)[AttnGenCfg<DP>::kChunks]) {
#pragma unroll
  for (int i = 0; i < AttnGenCfg<DP>::kChunks; i++) {
    int const c = t + i * 256;
    int const row = c / (DP / 8), ch = c % (DP / 8);
    *reinterpret_cast<u32x4 *>(tile + row * AttnGenCfg<DP>::kStride + ch * 8) = r[i];
  }
}

// --------------------------------------------------------------------------
// forward: workgroup = 128 query rows of one (batch, head), 32 per wave
// --------------------------------------------------------------------------
template <int DP>
__global__ __launch_bounds__(256) void attn_gen_fwd_kernel(AttnGenParams p) {
  using C = AttnGenCfg<DP>;
  __shared__ __attribute__((aligned(16))) bf16 Ks[2][C::kTile * C::kStride];
  __shared__ __attribute__((aligned(16))) bf16 Vs[2][C::kTile * C::kStride];
  int const t = threadIdx.x, lane = t & 63, h32 = lane >> 5;
  int const wave = __builtin_amdgcn_readfirstlane(t >> 6);
  int const nqb = (p.Sq + C::kBlk - 1) / C::kBlk;
  int const hb = blockIdx.x % (p.H * p.B);
  int const qb = nqb - 1 - blockIdx.x / (p.H * p.B);  // heaviest causal blocks first
  int const head = hb % p.H, b = hb / p.H;
  int const q0 = qb * C::kBlk;
  int const qrow = q0 + wave * 32 + (lane & 31);
  bf16 const *qp = p.q + (int64_t)b * p.q_bs + (int64_t)head * p.Dq;
  bf16 const *kp = p.k + (int64_t)b * p.k_bs + (int64_t)head * p.Dq;
  bf16 const *vp = p.v + (int64_t)b * p.v_bs + (int64_t)head * p.Dv;

  bf16x8 qf[DP / 16];
  gen_load_owned<DP>(qp + (int64_t)min(qrow, p.Sq - 1) * p.q_ss, p.Dq, h32, qf);

  int kv_end = p.Skv;
  if (p.causal) kv_end = min(p.Skv, q0 + C::kBlk);
  int const ntiles = (kv_end + C::kTile - 1) / C::kTile;

  f32x16 oacc[DP / 32];
#pragma unroll
  for (int i = 0; i < DP / 32; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) oacc[i][r] = 0.0f;
  float m_run = -INFINITY, l_run = 0.0f;

  u32x4 rk[C::kChunks], rv[C::kChunks];
  auto fetch = [&](int kv0) {
    gen_tile_gload<DP>(kp, p.k_ss, kv0, p.Skv - 1, p.Dq, t, rk);
    gen_tile_gload<DP>(vp, p.v_ss, kv0, p.Skv - 1, p.Dv, t, rv);
  };
  auto stash = [&](int buf) {
    gen_tile_lstore<DP>(Ks[buf], t, rk);
    gen_tile_lstore<DP>(Vs[buf], t, rv);
  };
  int const koff = lane_k_off(C::kStride, lane);
  int const toff = lane_tr_off(C::kStride, lane);
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
      bf16 const *kt = Ks[cur] + koff;
      bf16 const *vt = Vs[cur] + toff;
      // S^T: rows = keys of the tile, column = this lane's query
      f32x16 s;
#pragma unroll
      for (int r = 0; r < 16; r++) s[r] = 0.0f;
#pragma unroll
      for (int kk = 0; kk < DP / 16; kk++) {
        bf16x8 const kf = frag_k(kt, C::kStride, 0, kk * 16);
        s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[kk], s, 0, 0, 0);
      }
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
      mx = max_across_halves(mx) * p.scale_log2;
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
      bf16x8 const pf[2] = {pack8(pv), pack8(pv + 8)};
      l_run = l_run * alpha + sum;  // this lane's 16 of the 32 keys; the lane halves meet at the end
      m_run = m_new;
      if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
        for (int i = 0; i < DP / 32; i++)
#pragma unroll
          for (int r = 0; r < 16; r++) oacc[i][r] *= alpha;
      }
      // O^T += V^T P^T: A = V^T (rows d) through transposing loads, B = P^T
#pragma unroll
      for (int i = 0; i < DP / 32; i++) {
#pragma unroll
        for (int s2 = 0; s2 < 2; s2++) {
          bf16x8 const vf = frag_tr_acc(vt, C::kStride, 0, s2, i * 32);
          oacc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf[s2], oacc[i], 0, 0, 0);
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

  l_run += __shfl_xor(l_run, 32, 64);
  if (qrow < p.Sq) {
    float const inv = 1.0f / l_run;
    bf16 *op = p.out + (int64_t)b * p.o_bs + (int64_t)qrow * p.o_ss + (int64_t)head * p.Dv;
#pragma unroll
    for (int i = 0; i < DP / 32; i++) {
#pragma unroll
      for (int g = 0; g < 4; g++) {
        int const d = i * 32 + 8 * g + 4 * h32;
        if (d < p.Dv) {
          u32x2 w = {pack_bf16x2(oacc[i][4 * g] * inv, oacc[i][4 * g + 1] * inv),
                     pack_bf16x2(oacc[i][4 * g + 2] * inv, oacc[i][4 * g + 3] * inv)};
          *reinterpret_cast<u32x2 *>(op + d) = w;
        }
      }
    }
    if (h32 == 0 && p.lse != nullptr) {
      p.lse[((int64_t)b * p.H + head) * p.Sq + qrow] = (m_run + __log2f(l_run)) * kLn2;
    }
  }
}

// --------------------------------------------------------------------------
// backward (B): dQ, and delta = rowsum(O * dO) for its rows.  Runs first.
// --------------------------------------------------------------------------
template <int DP>
__global__ __launch_bounds__(256) void attn_gen_bwd_dq_kernel(AttnGenParams p) {
  using C = AttnGenCfg<DP>;
  __shared__ __attribute__((aligned(16))) bf16 Ks[2][C::kTile * C::kStride];
  __shared__ __attribute__((aligned(16))) bf16 Vs[2][C::kTile * C::kStride];
  int const t = threadIdx.x, lane = t & 63, h32 = lane >> 5;
  int const wave = __builtin_amdgcn_readfirstlane(t >> 6);
  int const nqb = (p.Sq + C::kBlk - 1) / C::kBlk;
  int const hb = blockIdx.x % (p.H * p.B);
  int const qb = nqb - 1 - blockIdx.x / (p.H * p.B);
  int const head = hb % p.H, b = hb / p.H;
  int const q0 = qb * C::kBlk;
  int const qrow = q0 + wave * 32 + (lane & 31);
  bf16 const *qp = p.q + (int64_t)b * p.q_bs + (int64_t)head * p.Dq;
  bf16 const *gp = p.d_o + (int64_t)b * p.o_bs + (int64_t)head * p.Dv;
  bf16 const *op = p.o + (int64_t)b * p.o_bs + (int64_t)head * p.Dv;
  bf16 const *kp = p.k + (int64_t)b * p.k_bs + (int64_t)head * p.Dq;
  bf16 const *vp = p.v + (int64_t)b * p.v_bs + (int64_t)head * p.Dv;

  bf16x8 qf[DP / 16], gf[DP / 16];
  float lse2, delta_s;  // delta_s = delta * scale
  {
    int const r = min(qrow, p.Sq - 1);
    gen_load_owned<DP>(qp + (int64_t)r * p.q_ss, p.Dq, h32, qf);
    gen_load_owned<DP>(gp + (int64_t)r * p.o_ss, p.Dv, h32, gf);
    lse2 = p.lse[((int64_t)b * p.H + head) * p.Sq + r] * kLog2e;
    // delta of this lane's row: the lane holds 8 of every 16 columns, its partner l ^ 32 the rest
    float part = 0.0f;
#pragma unroll
    for (int kk = 0; kk < DP / 16; kk++) {
      union {
        u32x4 u;
        bf16x8 v;
      } of;
      of.u = load8_or_zero(op + (int64_t)r * p.o_ss, kk * 16 + h32 * 8, p.Dv);
#pragma unroll
      for (int e = 0; e < 8; e++) part += (float)of.v[e] * (float)gf[kk][e];
    }
    float const delta = part + __shfl_xor(part, 32, 64);
    if (h32 == 0 && qrow < p.Sq) p.delta[((int64_t)b * p.H + head) * p.Sq + qrow] = delta;
    delta_s = delta * p.scale;
  }
  f32x16 dq[DP / 32];
#pragma unroll
  for (int i = 0; i < DP / 32; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) dq[i][r] = 0.0f;

  int kv_end = p.Skv;
  if (p.causal) kv_end = min(p.Skv, q0 + C::kBlk);
  int const ntiles = (kv_end + C::kTile - 1) / C::kTile;

  u32x4 rk[C::kChunks], rv[C::kChunks];
  auto fetch = [&](int kt0) {
    gen_tile_gload<DP>(kp, p.k_ss, kt0, p.Skv - 1, p.Dq, t, rk);
    gen_tile_gload<DP>(vp, p.v_ss, kt0, p.Skv - 1, p.Dv, t, rv);
  };
  auto stash = [&](int buf) {
    gen_tile_lstore<DP>(Ks[buf], t, rk);
    gen_tile_lstore<DP>(Vs[buf], t, rv);
  };
  int const koff = lane_k_off(C::kStride, lane);
  int const toff = lane_tr_off(C::kStride, lane);
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
      bf16 const *kk_ = Ks[cur] + koff, *vk_ = Vs[cur] + koff, *ktr = Ks[cur] + toff;
      // S^T = K Q^T, dP^T = V dO^T: rows = keys of the tile, column = this lane's query
      f32x16 s, dp;
#pragma unroll
      for (int r = 0; r < 16; r++) {
        s[r] = 0.0f;
        dp[r] = 0.0f;
      }
#pragma unroll
      for (int kk = 0; kk < DP / 16; kk++) {
        bf16x8 const ka = frag_k(kk_, C::kStride, 0, kk * 16);
        s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka, qf[kk], s, 0, 0, 0);
        bf16x8 const va = frag_k(vk_, C::kStride, 0, kk * 16);
        dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va, gf[kk], dp, 0, 0, 0);
      }
      float dsv[16];
#pragma unroll
      for (int r = 0; r < 16; r++) {
        int const kv = kt0 + 8 * (r >> 2) + 4 * h32 + (r & 3);
        float const e = __builtin_amdgcn_exp2f(__builtin_fmaf(s[r], p.scale_log2, -lse2));
        bool const masked = kv >= p.Skv || (p.causal && kv > qrow);
        dsv[r] = masked ? 0.0f : e * __builtin_fmaf(dp[r], p.scale, -delta_s);
      }
      // dQ^T += K^T dS^T: A = K^T (rows d) through transposing loads, B = dS^T
#pragma unroll
      for (int s2 = 0; s2 < 2; s2++) {
        bf16x8 const db = pack8(dsv + 8 * s2);
#pragma unroll
        for (int i = 0; i < DP / 32; i++) {
          bf16x8 const ka = frag_tr_acc(ktr, C::kStride, 0, s2, i * 32);
          dq[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka, db, dq[i], 0, 0, 0);
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
    bf16 *dqp = p.dq + (int64_t)b * p.q_bs + (int64_t)qrow * p.q_ss + (int64_t)head * p.Dq;
#pragma unroll
    for (int i = 0; i < DP / 32; i++) {
#pragma unroll
      for (int g = 0; g < 4; g++) {
        int const d = i * 32 + 8 * g + 4 * h32;
        if (d < p.Dq) {
          u32x2 w = {pack_bf16x2(dq[i][4 * g], dq[i][4 * g + 1]), pack_bf16x2(dq[i][4 * g + 2], dq[i][4 * g + 3])};
          *reinterpret_cast<u32x2 *>(dqp + d) = w;
        }
      }
    }
  }
}

// --------------------------------------------------------------------------
// backward (A): dK, dV.  Workgroup owns 128 key rows, streams query tiles.
// WHAT: bit 0 = produce dV, bit 1 = produce dK.
// --------------------------------------------------------------------------
template <int DP, int WHAT>
__global__ __launch_bounds__(256) void attn_gen_bwd_dkdv_kernel(AttnGenParams p) {
  using C = AttnGenCfg<DP>;
  constexpr bool kDV = (WHAT & 1) != 0, kDK = (WHAT & 2) != 0;
  __shared__ __attribute__((aligned(16))) bf16 Qs[2][C::kTile * C::kStride];
  __shared__ __attribute__((aligned(16))) bf16 Gs[2][C::kTile * C::kStride];  // dO
  __shared__ __attribute__((aligned(16))) float Ls[2][C::kTile], Ds[2][C::kTile];
  int const t = threadIdx.x, lane = t & 63, h32 = lane >> 5;
  int const wave = __builtin_amdgcn_readfirstlane(t >> 6);
  int const hb = blockIdx.x % (p.H * p.B);
  int const head = hb % p.H, b = hb / p.H;
  int const kv0 = (blockIdx.x / (p.H * p.B)) * C::kBlk;
  int const kvrow = kv0 + wave * 32 + (lane & 31);
  bf16 const *qp = p.q + (int64_t)b * p.q_bs + (int64_t)head * p.Dq;
  bf16 const *gp = p.d_o + (int64_t)b * p.o_bs + (int64_t)head * p.Dv;
  bf16 const *kp = p.k + (int64_t)b * p.k_bs + (int64_t)head * p.Dq;
  bf16 const *vp = p.v + (int64_t)b * p.v_bs + (int64_t)head * p.Dv;
  float const *lsep = p.lse + ((int64_t)b * p.H + head) * p.Sq;
  float const *delp = p.delta + ((int64_t)b * p.H + head) * p.Sq;

  bf16x8 kf[DP / 16];
  bf16x8 vf[kDK ? DP / 16 : 1];
  gen_load_owned<DP>(kp + (int64_t)min(kvrow, p.Skv - 1) * p.k_ss, p.Dq, h32, kf);
  if constexpr (kDK) gen_load_owned<DP>(vp + (int64_t)min(kvrow, p.Skv - 1) * p.v_ss, p.Dv, h32, vf);
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

  u32x4 rq[C::kChunks], rg[C::kChunks];
  float rl = 0.0f, rd = 0.0f;
  auto gload = [&](int qt0) {
    gen_tile_gload<DP>(qp, p.q_ss, qt0, p.Sq - 1, p.Dq, t, rq);
    gen_tile_gload<DP>(gp, p.o_ss, qt0, p.Sq - 1, p.Dv, t, rg);
    int const gr = min(qt0 + (t & (C::kTile - 1)), p.Sq - 1);
    rl = lsep[gr] * kLog2e;
    rd = delp[gr];
  };
  auto lstore = [&](int buf) {
    gen_tile_lstore<DP>(Qs[buf], t, rq);
    gen_tile_lstore<DP>(Gs[buf], t, rg);
    if (t < C::kTile) {
      Ls[buf][t] = rl;
      Ds[buf][t] = rd * p.scale;  // delta * scale, so dS is one fma and one multiply per element
    }
  };
  int const koff = lane_k_off(C::kStride, lane);
  int const toff = lane_tr_off(C::kStride, lane);
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
      bf16 const *qk = Qs[cur] + koff, *gk = Gs[cur] + koff;
      bf16 const *qtr = Qs[cur] + toff, *gtr = Gs[cur] + toff;
      // S = Q K^T and dP = dO V^T: rows = queries of the tile, column = this lane's key
      f32x16 s, dp;
#pragma unroll
      for (int r = 0; r < 16; r++) {
        s[r] = 0.0f;
        dp[r] = 0.0f;
      }
#pragma unroll
      for (int kk = 0; kk < DP / 16; kk++) {
        bf16x8 const qa = frag_k(qk, C::kStride, 0, kk * 16);
        s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qa, kf[kk], s, 0, 0, 0);
        if constexpr (kDK) {
          bf16x8 const ga = frag_k(gk, C::kStride, 0, kk * 16);
          dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ga, vf[kk], dp, 0, 0, 0);
        }
      }
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
      // dV += P^T dO ; dK += dS^T Q.  A = the accumulator re-used (row = key), B = dO / Q read
      // with the matching reduction order (k = query)
#pragma unroll
      for (int s2 = 0; s2 < 2; s2++) {
        bf16x8 const pa = pack8(pv + 8 * s2);
        bf16x8 const da = pack8(dsv + 8 * s2);
#pragma unroll
        for (int i = 0; i < DP / 32; i++) {
          if constexpr (kDV) {
            bf16x8 const gb = frag_tr_acc(gtr, C::kStride, 0, s2, i * 32);
            dv[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(pa, gb, dv[i], 0, 0, 0);
          }
          if constexpr (kDK) {
            bf16x8 const qb = frag_tr_acc(qtr, C::kStride, 0, s2, i * 32);
            dk[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(da, qb, dk[i], 0, 0, 0);
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

  // dK / dV accumulators: row = key (8*(r/4) + 4*h + r%4 of this wave's 32), column = d, so a
  // lane holds one column of 16 rows.  Each wave turns its 32 x DP block around in LDS (the
  // streamed tiles are done with) and writes whole 16-byte pieces of rows.
  __syncthreads();
  constexpr int kOutStride = DP + 8;
  bf16 *const stage = (wave < 2 ? &Qs[0][0] : &Gs[0][0]) + (wave & 1) * 32 * kOutStride;
  static_assert(2 * 32 * kOutStride <= 2 * C::kTile * C::kStride, "staging fits the tile buffers");
  auto write_out = [&](f32x16 const (&acc)[DP / 32], bf16 *out, int64_t row_stride, int D) {
#pragma unroll
    for (int i = 0; i < DP / 32; i++) {
#pragma unroll
      for (int r = 0; r < 16; r++) {
        int const row = 8 * (r >> 2) + 4 * h32 + (r & 3);
        VecIO<bf16>::store1(stage + row * kOutStride + i * 32 + (lane & 31), acc[i][r]);
      }
    }
    // LDS operations of one wave complete in order: the reads below see the writes above
#pragma unroll
    for (int k = 0; k < 32 * (DP / 8) / 64; k++) {
      int const c = lane + k * 64;
      int const row = c / (DP / 8), ch = c % (DP / 8);
      u32x4 const v = *reinterpret_cast<u32x4 const *>(stage + row * kOutStride + ch * 8);
      int const grow = kv0 + wave * 32 + row;
      if (grow < p.Skv && ch * 8 < D) *reinterpret_cast<u32x4 *>(out + (int64_t)grow * row_stride + ch * 8) = v;
    }
  };
  if constexpr (kDK) write_out(dk, p.dk + (int64_t)b * p.k_bs + (int64_t)head * p.Dq, p.k_ss, p.Dq);
  if constexpr (kDV) write_out(dv, p.dv + (int64_t)b * p.v_bs + (int64_t)head * p.Dv, p.v_ss, p.Dv);
}

static int check_desc_gen(char const *who, ffk_attention_desc_t const *d) {
  int64_t const dq = d->head_dim, dv = d->v_head_dim > 0 ? d->v_head_dim : d->head_dim;
  FFK_REQUIRE(dq > 0 && dq <= 256 && dq % 8 == 0 && dv <= 256 && dv % 8 == 0,
              "%s: bf16 head_dim %lld / v_head_dim %lld not supported (multiples of 8 up to 256)", who,
              (long long)dq, (long long)dv);
  FFK_REQUIRE(d->q_seq_stride >= d->heads * dq && d->k_seq_stride >= d->heads * dq &&
                  d->v_seq_stride >= d->heads * dv && d->o_seq_stride >= d->heads * dv,
              "%s: sequence stride smaller than heads * head_dim", who);
  return FFK_OK;
}

static AttnGenParams make_gen_params(ffk_attention_desc_t const *d) {
  AttnGenParams p = {};
  p.B = (int)d->batch; p.H = (int)d->heads; p.Sq = (int)d->seq_q; p.Skv = (int)d->seq_kv;
  p.Dq = (int)d->head_dim;
  p.Dv = (int)(d->v_head_dim > 0 ? d->v_head_dim : d->head_dim);
  p.q_bs = d->q_batch_stride; p.q_ss = d->q_seq_stride;
  p.k_bs = d->k_batch_stride; p.k_ss = d->k_seq_stride;
  p.v_bs = d->v_batch_stride; p.v_ss = d->v_seq_stride;
  p.o_bs = d->o_batch_stride; p.o_ss = d->o_seq_stride;
  p.scale = d->scale;
  p.scale_log2 = d->scale * kLog2e;
  p.causal = d->causal;
  return p;
}

#define FFK_ATTN_GEN_DISPATCH(D_, CALL)                                        \
  do {                                                                         \
    if ((D_) <= 64) { CALL(64); }                                              \
    else if ((D_) <= 128) { CALL(128); }                                       \
    else { CALL(256); }                                                        \
  } while (0)

// shapes, strides and alignment other than the head sizes are checked by the caller (attention.hip)
int attention_bf16_general_forward(hipStream_t st, ffk_attention_desc_t const *d, void const *q, void const *k,
                                   void const *v, void *o, float *lse) {
  int rc = check_desc_gen("attention_forward", d);
  if (rc != FFK_OK) return rc;
  AttnGenParams p = make_gen_params(d);
  p.q = static_cast<bf16 const *>(q);
  p.k = static_cast<bf16 const *>(k);
  p.v = static_cast<bf16 const *>(v);
  p.out = static_cast<bf16 *>(o);
  p.lse = lse;
  unsigned const grid = (unsigned)(ceil_div(p.Sq, 128) * p.H * p.B);
  int const dmax = p.Dq > p.Dv ? p.Dq : p.Dv;
#define CALL(DP_) attn_gen_fwd_kernel<DP_><<<grid, 256, 0, st>>>(p)
  FFK_ATTN_GEN_DISPATCH(dmax, CALL);
#undef CALL
  FFK_CHECK_LAUNCH();
  return FFK_OK;
}

template <int DP>
static void launch_gen_backward(hipStream_t st, AttnGenParams const &p, unsigned gkv, unsigned gq) {
  // dQ first: it leaves delta in memory for the dK/dV kernel
  attn_gen_bwd_dq_kernel<DP><<<gq, 256, 0, st>>>(p);
  if constexpr (DP <= 128) {
    attn_gen_bwd_dkdv_kernel<DP, 3><<<gkv, 256, 0, st>>>(p);
  } else {
    attn_gen_bwd_dkdv_kernel<DP, 1><<<gkv, 256, 0, st>>>(p);
    attn_gen_bwd_dkdv_kernel<DP, 2><<<gkv, 256, 0, st>>>(p);
  }
}

int attention_bf16_general_backward(hipStream_t st, ffk_attention_desc_t const *d, void const *q, void const *k,
                                    void const *v, void const *o, void const *d_o, float const *lse,
                                    float *delta, void *dq, void *dk, void *dv) {
  int rc = check_desc_gen("attention_backward", d);
  if (rc != FFK_OK) return rc;
  AttnGenParams p = make_gen_params(d);
  p.q = static_cast<bf16 const *>(q);
  p.k = static_cast<bf16 const *>(k);
  p.v = static_cast<bf16 const *>(v);
  p.o = static_cast<bf16 const *>(o);
  p.d_o = static_cast<bf16 const *>(d_o);
  p.lse = const_cast<float *>(lse);
  p.delta = delta;
  p.dq = static_cast<bf16 *>(dq);
  p.dk = static_cast<bf16 *>(dk);
  p.dv = static_cast<bf16 *>(dv);
  unsigned const gkv = (unsigned)(ceil_div(p.Skv, 128) * p.H * p.B);
  unsigned const gq = (unsigned)(ceil_div(p.Sq, 128) * p.H * p.B);
  int const dmax = p.Dq > p.Dv ? p.Dq : p.Dv;
#define CALL(DP_) launch_gen_backward<DP_>(st, p, gkv, gq)
  FFK_ATTN_GEN_DISPATCH(dmax, CALL);
#undef CALL
  FFK_CHECK_LAUNCH();
  return FFK_OK;
}

}  // namespace ffk
