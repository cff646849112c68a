// Fused (flash-style) attention for gfx950, bf16 operands / fp32 accumulation.
//
// The reference hands Q, K, V to cudnnMultiHeadAttnForward / BackwardData
// (lib/kernels/src/cuda/ops/attention_kernels.cu:224,261), which materialise
// the seq x seq score matrix.  Here scores never leave the CU:
//
//  forward   one workgroup = 128 query rows of one (batch, head); each of its
//            4 wavefronts owns 32 rows.  Scores are computed transposed,
//            S^T = K Q^T, so that a lane owns one query row's column of the
//            MFMA accumulator: the running max / sum are lane-local and the
//            probabilities feed the P V product straight from registers.
//            V is staged in LDS as it lies in memory and read with the
//            transposing LDS load.
//  backward  two kernels, no atomics, deterministic:
//            (A) one workgroup = 128 key/value rows, loops over query tiles and
//                accumulates dK, dV in registers;
//            (B) one workgroup = 128 query rows, loops over key tiles and
//                accumulates dQ in registers.
//            Both recompute P from the saved log-sum-exp.  (B) runs first: it also computes
//            delta = rowsum(O * dO) for its rows and leaves it in memory for (A).
//
// MFMA 32x32x16 bf16 register layouts used throughout (l = lane):
//   A operand: row l%32, k = 8*(l/32) .. +7      B operand: column l%32, same k
//   accumulator element r: row 8*(r/4) + 4*(l/32) + r%4, column l%32.
// When an accumulator tile is re-used as an operand of the next product, its
// 8 values r = 8s .. 8s+7 are taken as the k-slots of step s; the other operand
// is then loaded with the same permutation of the reduction index, which the
// transposing load does for free.
#include "attention_common.h"
#include <type_traits>

namespace ffk {

template <int D>
struct AttnCfg {
  static constexpr int kBQ = 128;          // query rows per workgroup (forward, dQ)
  static constexpr int kBKV = 64;          // key rows per LDS tile (forward, dQ)
  static constexpr int kKStride = D + 8;   // K tile row stride (b128 reads)
  static constexpr int kVStride = D + 32;  // V tile row stride (transposing reads)
  static constexpr int kChunks = kBKV * D / 8 / 256;  // 16-byte chunks per thread
};

// --------------------------------------------------------------------------
// forward
// --------------------------------------------------------------------------
template <int D>
__global__ __launch_bounds__(256, 2) void attn_fwd_kernel(AttnParams p) {
  using C = AttnCfg<D>;
  __shared__ __attribute__((aligned(16))) bf16 Ks[2][C::kBKV * C::kKStride];
  __shared__ __attribute__((aligned(16))) bf16 Vs[2][C::kBKV * C::kVStride];
  int const t = threadIdx.x, lane = t & 63, h32 = lane >> 5;
  // the wave index as a scalar: tile-level decisions taken from it are branches, not lane masks
  int const wave = __builtin_amdgcn_readfirstlane(t >> 6);
  // 1-D grid ordered so that, under a causal mask, the heaviest (latest) query
  // blocks of every (batch, head) are dispatched first and light ones fill the tail.
  int const nqb = (p.Sq + C::kBQ - 1) / C::kBQ;
  int const hb = blockIdx.x % (p.H * p.B);
  int const qb = nqb - 1 - blockIdx.x / (p.H * p.B);
  int const head = hb % p.H, b = hb / p.H;
  int const q0 = qb * C::kBQ;
  int const qrow = q0 + wave * 32 + (lane & 31);  // this lane's query row
  bf16 const *qp = p.q + (int64_t)b * p.q_bs + (int64_t)head * D;
  bf16 const *kp = p.k + (int64_t)b * p.k_bs + (int64_t)head * D;
  bf16 const *vp = p.v + (int64_t)b * p.v_bs + (int64_t)head * D;

  // Q as the B operand of S^T = K Q^T: column = query row, k = d.
  bf16x8 qf[D / 16];
  {
    int const r = min(qrow, p.Sq - 1);
#pragma unroll
    for (int kk = 0; kk < D / 16; kk++) {
      qf[kk] = *reinterpret_cast<bf16x8 const *>(qp + (int64_t)r * p.q_ss + kk * 16 + h32 * 8);
    }
  }

  int kv_end = p.Skv;
  if (p.causal) kv_end = min(p.Skv, q0 + C::kBQ);
  int const ntiles = (kv_end + C::kBKV - 1) / C::kBKV;

  u32x4 rk[C::kChunks], rv[C::kChunks];
  auto gload = [&](int kv0) {
#pragma unroll
    for (int i = 0; i < C::kChunks; i++) {
      int c = t + i * 256;
      int row = c / (D / 8), ch = c % (D / 8);
      int gr = min(kv0 + row, p.Skv - 1);
      rk[i] = *reinterpret_cast<u32x4 const *>(kp + (int64_t)gr * p.k_ss + ch * 8);
      rv[i] = *reinterpret_cast<u32x4 const *>(vp + (int64_t)gr * p.v_ss + ch * 8);
    }
  };
  auto lstore = [&](int buf) {
#pragma unroll
    for (int i = 0; i < C::kChunks; i++) {
      int c = t + i * 256;
      int row = c / (D / 8), ch = c % (D / 8);
      *reinterpret_cast<u32x4 *>(&Ks[buf][row * C::kKStride + ch * 8]) = rk[i];
      *reinterpret_cast<u32x4 *>(&Vs[buf][row * C::kVStride + ch * 8]) = rv[i];
    }
  };

  f32x16 oacc[D / 32];
#pragma unroll
  for (int i = 0; i < D / 32; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) oacc[i][r] = 0.0f;
  float m_run = -INFINITY, l_run = 0.0f;

  int const koff = lane_k_off(C::kKStride, lane);
  int const voff = lane_tr_off(C::kVStride, lane);
  gload(0);
  lstore(0);
  __syncthreads();
  int cur = 0;
  for (int it = 0; it < ntiles; it++) {
    int const kv0 = it * C::kBKV;
    bool const more = it + 1 < ntiles;
    if (more) gload(kv0 + C::kBKV);

    // A wave whose rows all lie before this tile (causal) has nothing to add.
    bool const active = !p.causal || kv0 <= q0 + wave * 32 + 31;
    if (active) {
      bf16 const *kt = Ks[cur] + koff;
      bf16 const *vt = Vs[cur] + voff;
      // S^T tiles: rows = keys (32 per tile), columns = this wave's queries.
      f32x16 s[C::kBKV / 32];
#pragma unroll
      for (int j = 0; j < C::kBKV / 32; j++) {
#pragma unroll
        for (int r = 0; r < 16; r++) s[j][r] = 0.0f;
#pragma unroll
        for (int kk = 0; kk < D / 16; kk++) {
          bf16x8 kf = frag_k(kt, C::kKStride, j * 32, kk * 16);
          s[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[kk], s[j], 0, 0, 0);
        }
      }
      // mask (only tiles that straddle the end of the keys or the causal diagonal), running
      // max of the raw scores (the scale is positive, so it commutes with the max)
      bool const need_mask = (kv0 + C::kBKV > p.Skv) || (p.causal && kv0 + C::kBKV - 1 > q0 + wave * 32);
      if (need_mask) {
#pragma unroll
        for (int j = 0; j < C::kBKV / 32; j++) {
#pragma unroll
          for (int r = 0; r < 16; r++) {
            int kv = kv0 + j * 32 + 8 * (r >> 2) + 4 * h32 + (r & 3);
            if (kv >= p.Skv || (p.causal && kv > qrow)) s[j][r] = -INFINITY;
          }
        }
      }
      float mx = -INFINITY;
#pragma unroll
      for (int j = 0; j < C::kBKV / 32; j++) {
#pragma unroll
        for (int r = 0; r < 16; r++) mx = fmaxf(mx, s[j][r]);
      }
      mx = max_across_halves(mx) * p.scale_log2;  // a lane swap, no trip through LDS
      float const m_new = fmaxf(m_run, mx);
      // m_new is finite: key 0 is visible to every query and tile 0 comes first.
      float const alpha = __builtin_amdgcn_exp2f(m_run - m_new);
      float sum = 0.0f;
      bf16x8 pf[C::kBKV / 16];
#pragma unroll
      for (int j = 0; j < C::kBKV / 32; j++) {
        float pv[16];
#pragma unroll
        for (int r = 0; r < 16; r++) {
          float e = __builtin_amdgcn_exp2f(__builtin_fmaf(s[j][r], p.scale_log2, -m_new));
          pv[r] = e;
          sum += e;
        }
        pf[2 * j] = pack8(pv);
        pf[2 * j + 1] = pack8(pv + 8);
      }
      l_run = l_run * alpha + sum;  // this lane's 16 of every 32 keys; the two lane halves meet at the end
      m_run = m_new;
      // Rescale the running output only when some row's maximum moved.
      if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
        for (int i = 0; i < D / 32; i++)
#pragma unroll
          for (int r = 0; r < 16; r++) oacc[i][r] *= alpha;
      }
      // O^T += V^T P^T : A = V^T (rows d) via transposing loads, B = P^T.
#pragma unroll
      for (int i = 0; i < D / 32; i++) {
#pragma unroll
        for (int j = 0; j < C::kBKV / 32; j++) {
#pragma unroll
          for (int s2 = 0; s2 < 2; s2++) {
            bf16x8 vf = frag_tr_acc(vt, C::kVStride, j * 32, s2, i * 32);
            oacc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf[2 * j + s2], oacc[i], 0, 0, 0);
          }
        }
      }
    }
    if (more) lstore(cur ^ 1);
    __syncthreads();
    cur ^= 1;
  }

  l_run += __shfl_xor(l_run, 32, 64);
  if (qrow < p.Sq) {
    float const inv = 1.0f / l_run;
    bf16 *op = p.o + (int64_t)b * p.o_bs + (int64_t)qrow * p.o_ss + (int64_t)head * D;
#pragma unroll
    for (int i = 0; i < D / 32; i++) {
#pragma unroll
      for (int g = 0; g < 4; g++) {
        int d = i * 32 + 8 * g + 4 * h32;
        u32x2 w = {pack_bf16x2(oacc[i][4 * g] * inv, oacc[i][4 * g + 1] * inv),
                   pack_bf16x2(oacc[i][4 * g + 2] * inv, oacc[i][4 * g + 3] * inv)};
        *reinterpret_cast<u32x2 *>(op + d) = w;
      }
    }
    if (h32 == 0 && p.lse != nullptr) {
      p.lse[((int64_t)b * p.H + head) * p.Sq + qrow] = (m_run + __log2f(l_run)) * kLn2;
    }
  }
}

// --------------------------------------------------------------------------
// backward
// --------------------------------------------------------------------------

template <int D>
struct AttnBwdCfg {
  static constexpr int kBlk = 128;         // rows owned by a workgroup
  static constexpr int kTile = 32;         // rows of the streamed operand per step
  static constexpr int kStride = D + 40;   // serves b128 and transposing reads
  static constexpr int kChunks = kTile * D / 8 / 256;
  static_assert(kTile * D / 8 % 256 == 0, "tile chunks");
};

// (B) dQ: workgroup owns 128 query rows (32 per wave), streams key tiles.
template <int D>
__global__ __launch_bounds__(256) void attn_bwd_dq_kernel(AttnBwdParams p) {
  using C = AttnBwdCfg<D>;
  __shared__ __attribute__((aligned(16))) bf16 Ks[2][C::kTile * C::kStride];
  __shared__ __attribute__((aligned(16))) bf16 Vs[2][C::kTile * C::kStride];
  int const t = threadIdx.x, lane = t & 63, h32 = lane >> 5;
  // the wave index as a scalar: tile-level decisions taken from it are branches, not lane masks
  int const wave = __builtin_amdgcn_readfirstlane(t >> 6);
  int const nqb = (p.Sq + C::kBlk - 1) / C::kBlk;
  int const hb = blockIdx.x % (p.H * p.B);
  int const qb = nqb - 1 - blockIdx.x / (p.H * p.B);
  int const head = hb % p.H, b = hb / p.H;
  int const q0 = qb * C::kBlk;
  int const qrow = q0 + wave * 32 + (lane & 31);
  bf16 const *qp = p.q + (int64_t)b * p.q_bs + (int64_t)head * D;
  bf16 const *gp = p.d_o + (int64_t)b * p.o_bs + (int64_t)head * D;
  bf16 const *kp = p.k + (int64_t)b * p.k_bs + (int64_t)head * D;
  bf16 const *vp = p.v + (int64_t)b * p.v_bs + (int64_t)head * D;

  bf16x8 qf[D / 16], gf[D / 16];
  float lse2, delta_s;  // delta_s = delta * scale
  {
    int const r = min(qrow, p.Sq - 1);
#pragma unroll
    for (int kk = 0; kk < D / 16; kk++) {
      qf[kk] = *reinterpret_cast<bf16x8 const *>(qp + (int64_t)r * p.q_ss + kk * 16 + h32 * 8);
      gf[kk] = *reinterpret_cast<bf16x8 const *>(gp + (int64_t)r * p.o_ss + kk * 16 + h32 * 8);
    }
    lse2 = p.lse[((int64_t)b * p.H + head) * p.Sq + r] * kLog2e;
    // delta = sum_d O * dO of this lane's row: the lane holds half of the row's d (8 of every 16),
    // its partner l ^ 32 the other half.  The kernel that owns a query row is the one place that
    // has the row's dO in registers anyway; it leaves delta in memory for the dK/dV kernel, which
    // runs after it.
    bf16 const *op = p.o + (int64_t)b * p.o_bs + (int64_t)head * D;
    float part = 0.0f;
#pragma unroll
    for (int kk = 0; kk < D / 16; kk++) {
      bf16x8 const of = *reinterpret_cast<bf16x8 const *>(op + (int64_t)r * p.o_ss + kk * 16 + h32 * 8);
#pragma unroll
      for (int e = 0; e < 8; e++) part += (float)of[e] * (float)gf[kk][e];
    }
    float const delta = part + __shfl_xor(part, 32, 64);
    if (h32 == 0 && qrow < p.Sq) p.delta[((int64_t)b * p.H + head) * p.Sq + qrow] = delta;
    delta_s = delta * p.scale;
  }
  f32x16 dq[D / 32];
#pragma unroll
  for (int i = 0; i < D / 32; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) dq[i][r] = 0.0f;

  int kv_end = p.Skv;
  if (p.causal) kv_end = min(p.Skv, q0 + C::kBlk);
  int const ntiles = (kv_end + C::kTile - 1) / C::kTile;

  // Two register sets, loads two steps ahead of their use (see the dK/dV kernel).
  u32x4 rk[2][C::kChunks], rv[2][C::kChunks];
  auto gload = [&](int kt0, auto set_tag) {
    constexpr int R = decltype(set_tag)::value;
#pragma unroll
    for (int i = 0; i < C::kChunks; i++) {
      int c = t + i * 256;
      int row = c / (D / 8), ch = c % (D / 8);
      int gr = min(kt0 + row, p.Skv - 1);
      rk[R][i] = *reinterpret_cast<u32x4 const *>(kp + (int64_t)gr * p.k_ss + ch * 8);
      rv[R][i] = *reinterpret_cast<u32x4 const *>(vp + (int64_t)gr * p.v_ss + ch * 8);
    }
  };
  auto lstore = [&](auto set_tag) {
    constexpr int R = decltype(set_tag)::value;
#pragma unroll
    for (int i = 0; i < C::kChunks; i++) {
      int c = t + i * 256;
      int row = c / (D / 8), ch = c % (D / 8);
      *reinterpret_cast<u32x4 *>(&Ks[R][row * C::kStride + ch * 8]) = rk[R][i];
      *reinterpret_cast<u32x4 *>(&Vs[R][row * C::kStride + ch * 8]) = rv[R][i];
    }
  };
  using Set0 = std::integral_constant<int, 0>;
  using Set1 = std::integral_constant<int, 1>;

  int const koff = lane_k_off(C::kStride, lane);
  int const toff = lane_tr_off(C::kStride, lane);
  gload(0, Set0{});
  lstore(Set0{});
  gload(C::kTile, Set1{});  // unconditional, like every prefetch below (see the dK/dV kernel)
  __syncthreads();
  auto step = [&](int it, auto parity) {
    constexpr int cur = decltype(parity)::value;  // == it % 2
    int const kt0 = it * C::kTile;
    gload(kt0 + 2 * C::kTile, parity);
    bool const active = it < ntiles && (!p.causal || kt0 <= q0 + wave * 32 + 31);
    if (active) {
      bf16 const *kk_ = Ks[cur] + koff, *vk_ = Vs[cur] + koff, *ktr = Ks[cur] + toff;
      // S^T = K Q^T, dP^T = V dO^T: rows = keys of the tile, column = query.
      f32x16 s, dp;
#pragma unroll
      for (int r = 0; r < 16; r++) {
        s[r] = 0.0f;
        dp[r] = 0.0f;
      }
#pragma unroll
      for (int kk = 0; kk < D / 16; kk++) {
        bf16x8 ka = frag_k(kk_, C::kStride, 0, kk * 16);
        s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka, qf[kk], s, 0, 0, 0);
        bf16x8 va = frag_k(vk_, C::kStride, 0, kk * 16);
        dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va, gf[kk], dp, 0, 0, 0);
      }
      float dsv[16];
      bool const edge = kt0 + C::kTile > p.Skv || (p.causal && kt0 + C::kTile - 1 > q0 + wave * 32);
#pragma unroll
      for (int r = 0; r < 16; r++) {
        float const e = __builtin_amdgcn_exp2f(__builtin_fmaf(s[r], p.scale_log2, -lse2));
        dsv[r] = e * __builtin_fmaf(dp[r], p.scale, -delta_s);
      }
      if (edge) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
          int const kv = kt0 + 8 * (r >> 2) + 4 * h32 + (r & 3);
          bool const masked = kv >= p.Skv || (p.causal && kv > qrow);
          dsv[r] = masked ? 0.0f : dsv[r];
        }
      }
      // dQ^T += K^T dS^T : A = K^T (rows d) via transposing loads, B = dS^T.
#pragma unroll
      for (int s2 = 0; s2 < 2; s2++) {
        bf16x8 db = pack8(dsv + 8 * s2);
#pragma unroll
        for (int i = 0; i < D / 32; i++) {
          bf16x8 ka = frag_tr_acc(ktr, C::kStride, 0, s2, i * 32);
          dq[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka, db, dq[i], 0, 0, 0);
        }
      }
    }
    if (it + 1 < ntiles) lstore(std::integral_constant<int, cur ^ 1>{});
    __syncthreads();
  };
  // always in pairs (an odd count runs one idle step): the loop body then issues the same
  // loads whatever the tile count, which keeps the waits on them exact
  for (int it = 0; it < ntiles; it += 2) {
    step(it, Set0{});
    step(it + 1, Set1{});
  }

  if (qrow < p.Sq) {
    bf16 *dqp = p.dq + (int64_t)b * p.q_bs + (int64_t)qrow * p.q_ss + (int64_t)head * D;
#pragma unroll
    for (int i = 0; i < D / 32; i++) {
#pragma unroll
      for (int g = 0; g < 4; g++) {
        int d = i * 32 + 8 * g + 4 * h32;
        u32x2 w = {pack_bf16x2(dq[i][4 * g], dq[i][4 * g + 1]),
                   pack_bf16x2(dq[i][4 * g + 2], dq[i][4 * g + 3])};
        *reinterpret_cast<u32x2 *>(dqp + d) = w;
      }
    }
  }
}

// 64 query rows per wavefront (attention_fwd.hip)
hipError_t attention_bf16_forward_wide(hipStream_t st, AttnParams const &p, int head_dim);

// dK/dV with direct loads, one workgroup per CU: its three Q and three dO tile buffers take
// 48 KB (head size 64) or 96 KB (128) of LDS, and one wave per SIMD holds the accumulators (attention_bwd.hip)
hipError_t attention_bf16_dkdv(hipStream_t st, AttnBwdParams const &p, int head_dim);

// the fp32 core (attention_f32.hip)
int attention_f32_forward(hipStream_t st, ffk_attention_desc_t const *d, void const *q, void const *k,
                          void const *v, void *o, float *lse);
int attention_f32_backward(hipStream_t st, ffk_attention_desc_t const *d, void const *q, void const *k,
                           void const *v, void const *o, void const *d_o, float const *lse, float *delta,
                           void *dq, void *dk, void *dv);

// any multiple of 8 up to 256 for either head size (attention_gen.hip)
int attention_bf16_general_forward(hipStream_t st, ffk_attention_desc_t const *d, void const *q, void const *k,
                                   void const *v, void *o, float *lse);
int attention_bf16_general_backward(hipStream_t st, ffk_attention_desc_t const *d, void const *q, void const *k,
                                    void const *v, void const *o, void const *d_o, float const *lse,
                                    float *delta, void *dq, void *dk, void *dv);

// the kernels of this file and of attention_fwd.hip / attention_bwd.hip: one head size, 64 or 128
static bool tuned_head_size(ffk_attention_desc_t const *d) {
  return (d->head_dim == 64 || d->head_dim == 128) && (d->v_head_dim == 0 || d->v_head_dim == d->head_dim);
}

static int check_desc(char const *who, int dtype, ffk_attention_desc_t const *d) {
  FFK_REQUIRE(d != nullptr, "%s: NULL descriptor", who);
  // FLOAT was dispatched to the fp32 core before this check: what is left must be BF16
  FFK_REQUIRE(dtype == FFK_BF16, "%s: dtype %d not supported (the entry point takes FLOAT or BF16)", who, dtype);
  FFK_REQUIRE(d->head_dim > 0 && d->v_head_dim >= 0, "%s: bad head size", who);
  FFK_REQUIRE(d->batch > 0 && d->heads > 0 && d->seq_q > 0 && d->seq_kv > 0, "%s: bad shape", who);
  FFK_REQUIRE(d->batch * d->heads * ((d->seq_q > d->seq_kv ? d->seq_q : d->seq_kv) / 128 + 1) < (1ll << 31),
              "%s: too many workgroups", who);
  FFK_REQUIRE(d->seq_q < (1ll << 30) && d->seq_kv < (1ll << 30), "%s: sequence too long", who);
  FFK_REQUIRE(d->q_seq_stride % 8 == 0 && d->k_seq_stride % 8 == 0 && d->v_seq_stride % 8 == 0 &&
                  d->o_seq_stride % 8 == 0 && d->q_batch_stride % 8 == 0 && d->k_batch_stride % 8 == 0 &&
                  d->v_batch_stride % 8 == 0 && d->o_batch_stride % 8 == 0,
              "%s: strides must be multiples of 8 elements", who);
  if (tuned_head_size(d)) {
    FFK_REQUIRE(d->q_seq_stride >= d->heads * d->head_dim && d->k_seq_stride >= d->heads * d->head_dim &&
                    d->v_seq_stride >= d->heads * d->head_dim && d->o_seq_stride >= d->heads * d->head_dim,
                "%s: sequence stride smaller than heads * head_dim", who);
  }
  return FFK_OK;
}

}  // namespace ffk

using namespace ffk;

extern "C" int ffk_attention_forward(ffk_stream_t stream, int dtype,
                                     ffk_attention_desc_t const *d,
                                     void const *q, void const *k,
                                     void const *v, void *o, float *lse) {
  FFK_REQUIRE(d != nullptr, "attention_forward: NULL descriptor");
  FFK_REQUIRE(q && k && v && o, "attention_forward: NULL tensor");
  FFK_REQUIRE(aligned16(q) && aligned16(k) && aligned16(v) && aligned16(o),
              "attention_forward: tensors must be 16-byte aligned");
  if (dtype == FFK_FLOAT) return attention_f32_forward(as_stream(stream), d, q, k, v, o, lse);
  int rc = check_desc("attention_forward", dtype, d);
  if (rc != FFK_OK) return rc;
  if (!tuned_head_size(d)) return attention_bf16_general_forward(as_stream(stream), d, q, k, v, o, lse);
  AttnParams p;
  p.q = static_cast<bf16 const *>(q);
  p.k = static_cast<bf16 const *>(k);
  p.v = static_cast<bf16 const *>(v);
  p.o = static_cast<bf16 *>(o);
  p.lse = lse;
  p.B = (int)d->batch; p.H = (int)d->heads; p.Sq = (int)d->seq_q; p.Skv = (int)d->seq_kv;
  p.q_bs = d->q_batch_stride; p.q_ss = d->q_seq_stride;
  p.k_bs = d->k_batch_stride; p.k_ss = d->k_seq_stride;
  p.v_bs = d->v_batch_stride; p.v_ss = d->v_seq_stride;
  p.o_bs = d->o_batch_stride; p.o_ss = d->o_seq_stride;
  p.scale_log2 = d->scale * kLog2e;
  p.causal = d->causal;
  // 64 query rows per wavefront (256 per workgroup, one workgroup per CU) pay from about a
  // thousand keys on and when the problem still gives every CU a workgroup; below that the
  // kernel with 32 rows per wavefront and two workgroups per CU is ahead (config 2's 512 keys:
  // 18.5 against 19.4 us).
  int const variant = option(FFK_OPTION_ATTENTION_VARIANT);
  // (its direct loads address a 64-row tile with 32-bit byte offsets per lane)
  bool const wide_ok = p.k_ss < (int64_t(1) << 24) && p.v_ss < (int64_t(1) << 24);
  bool const wide = wide_ok && (variant == 2 || (variant == 0 && p.Skv >= 1024 &&
                                                 ceil_div(p.Sq, 256) * (int64_t)p.H * p.B >= kNumCU));
  if (wide) {
    FFK_HIP(attention_bf16_forward_wide(as_stream(stream), p, (int)d->head_dim));
    return FFK_OK;
  }
  dim3 grid((unsigned)(ceil_div(p.Sq, 128) * p.H * p.B));
  if (d->head_dim == 64) {
    attn_fwd_kernel<64><<<grid, 256, 0, as_stream(stream)>>>(p);
  } else {
    attn_fwd_kernel<128><<<grid, 256, 0, as_stream(stream)>>>(p);
  }
  FFK_CHECK_LAUNCH();
  return FFK_OK;
}

extern "C" int ffk_attention_backward(ffk_stream_t stream, int dtype,
                                      ffk_attention_desc_t const *d,
                                      void const *q, void const *k,
                                      void const *v, void const *o,
                                      void const *d_o, float const *lse,
                                      float *delta, void *dq, void *dk,
                                      void *dv) {
  FFK_REQUIRE(d != nullptr, "attention_backward: NULL descriptor");
  FFK_REQUIRE(q && k && v && o && d_o && lse && delta && dq && dk && dv,
              "attention_backward: NULL tensor");
  FFK_REQUIRE(aligned16(q) && aligned16(k) && aligned16(v) && aligned16(o) && aligned16(d_o) &&
                  aligned16(dq) && aligned16(dk) && aligned16(dv),
              "attention_backward: tensors must be 16-byte aligned");
  if (dtype == FFK_FLOAT) {
    return attention_f32_backward(as_stream(stream), d, q, k, v, o, d_o, lse, delta, dq, dk, dv);
  }
  int rc = check_desc("attention_backward", dtype, d);
  if (rc != FFK_OK) return rc;
  // (the tuned dK/dV kernel addresses a batch entry's rows with 32-bit byte offsets)
  int64_t const lim = int64_t(1) << 32;
  bool const offsets_fit = d->seq_q * d->q_seq_stride * 2 < lim && d->seq_q * d->o_seq_stride * 2 < lim &&
                           d->seq_kv * d->k_seq_stride * 2 < lim && d->seq_kv * d->v_seq_stride * 2 < lim;
  if (!tuned_head_size(d) || !offsets_fit) {
    return attention_bf16_general_backward(as_stream(stream), d, q, k, v, o, d_o, lse, delta, dq, dk, dv);
  }
  AttnBwdParams p;
  p.q = static_cast<bf16 const *>(q);
  p.k = static_cast<bf16 const *>(k);
  p.v = static_cast<bf16 const *>(v);
  p.o = static_cast<bf16 const *>(o);
  p.d_o = static_cast<bf16 const *>(d_o);
  p.lse = lse;
  p.delta = delta;
  p.dq = static_cast<bf16 *>(dq);
  p.dk = static_cast<bf16 *>(dk);
  p.dv = static_cast<bf16 *>(dv);
  p.B = (int)d->batch; p.H = (int)d->heads; p.Sq = (int)d->seq_q; p.Skv = (int)d->seq_kv;
  p.q_bs = d->q_batch_stride; p.q_ss = d->q_seq_stride;
  p.k_bs = d->k_batch_stride; p.k_ss = d->k_seq_stride;
  p.v_bs = d->v_batch_stride; p.v_ss = d->v_seq_stride;
  p.o_bs = d->o_batch_stride; p.o_ss = d->o_seq_stride;
  p.scale = d->scale;
  p.scale_log2 = d->scale * kLog2e;
  p.causal = d->causal;
  hipStream_t st = as_stream(stream);
  // dQ first: it computes delta for its rows and leaves it in `delta` for the dK/dV kernel
  dim3 gq((unsigned)(ceil_div(p.Sq, 128) * p.H * p.B));
  if (d->head_dim == 64) {
    attn_bwd_dq_kernel<64><<<gq, 256, 0, st>>>(p);
  } else {
    attn_bwd_dq_kernel<128><<<gq, 256, 0, st>>>(p);
  }
  FFK_CHECK_LAUNCH();
  FFK_HIP(attention_bf16_dkdv(st, p, (int)d->head_dim));
  FFK_CHECK_LAUNCH();
  return FFK_OK;
}
