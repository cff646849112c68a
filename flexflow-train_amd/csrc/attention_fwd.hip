// bf16 attention forward with 64 query rows per wavefront.
//
// One workgroup = 256 query rows of one (batch, head), 4 wavefronts of 64 rows,
// one workgroup per CU (one wavefront per SIMD, so a wavefront may use all 512
// registers).  A wavefront's rows are two halves of 32 (c = 0, 1).  Per tile of
// 64 keys both halves use the same K and V fragments, read from LDS once, and
// the wavefront overlaps the matrix pipe with the vector ALU itself:
//
//   phase 1   S_0 = K Q_0^T                      (MFMA, K fragments from LDS)
//   phase 2   S_1 = K Q_1^T   ||  softmax(S_0)    (MFMA || VALU)
//   phase 3   O_0 += V^T P_0  ||  softmax(S_1)    (MFMA, V fragments from LDS || VALU)
//   phase 4   O_1 += V^T P_1                     (MFMA)
//
// In phases 2 and 3 the MFMAs do not depend on the vector work next to them, and
// the scheduler is told to put one MFMA in front of every handful of vector
// instructions.  Layouts (scores transposed so that a lane owns a query's
// column, probabilities fed to the second product from registers) are those of
// the MFMA 32x32x16 bf16: A operand row l%32, k = 8*(l/32)..+7; B operand column
// l%32, same k; accumulator element r: row 8*(r/4) + 4*(l/32) + r%4, column l%32.
#include "attention_common.h"
#include "lds_dma.h"
#include <type_traits>

namespace ffk {

template <int D>
struct AttnFwdCfg {
  static constexpr int kBQ = 256;          // query rows per workgroup
  static constexpr int kBKV = 64;          // key rows per LDS tile
  // K and V tiles lie in LDS as they lie in memory, rows of D elements without padding: they
  // arrive by direct loads, which write a wave's 64 x 16 bytes contiguously.  Bank conflicts are
  // avoided by permuting the 16-byte chunks inside a row, on the fetching side:
  //   K (read with 16-byte loads, 16 lanes = 16 rows per cycle): chunk ^ kswz(row)
  //   V (read with transposing 8-byte loads, 32 lanes = 4 rows x 64 bytes per cycle):
  //     64-byte segment ^ vswz(row)
  static constexpr int kCPR = D / 8;                  // 16-byte chunks per row
  static constexpr int kLoads = kBKV * kCPR / 256;    // direct loads per thread, per tensor and tile
  static constexpr int kRowsPerLoad = 256 / kCPR;     // rows covered by one load of all 256 threads
  static constexpr int kTileElems = kBKV * D;
  __device__ static int kswz(int row) { return D == 128 ? (row & 15) : ((row >> 1) & 7); }
  __device__ static int vswz(int row) { return D == 128 ? (row & 3) : ((row >> 1) & 1); }
  static_assert(D == 64 || D == 128, "swizzles are written for these two");
};

// Online softmax of one half (32 queries x 64 keys: two score blocks, this lane's query column),
// cut into 16 units of a few vector instructions so that the caller can put one behind each MFMA
// of the product that runs next to it:
//   units 0..3   maximum of 8 of the lane's 32 scores each
//   unit  4      maximum over the two lane halves, new running maximum, factor for the old sums
//   units 5..15  exponentials: 3 scores each (the last takes 2), summed and packed as they come
struct SoftmaxHalf {
  static constexpr float kLazy = 8.0f;
  float mx, m_new, alpha, sum;
  float pv[2][16];
  // Ties a value to this point of the program.  Without it the optimizer moves a unit's
  // arithmetic to where its result is first needed, behind all the MFMAs it was to run next to.
  static __device__ __forceinline__ void here(float &x) { asm volatile("" : "+v"(x)); }
  template <int UNIT>
  __device__ __forceinline__ void unit(f32x16 const (&s)[2], float scale_log2, float m_run) {
    if constexpr (UNIT < 4) {
#pragma unroll
      for (int r = 4 * UNIT; r < 4 * UNIT + 4; r++) {
        // the running maximum and both blocks' scores in one three-operand maximum
        mx = (r == 0) ? fmaxf(s[0][r], s[1][r]) : fmaxf(fmaxf(mx, s[0][r]), s[1][r]);
      }
      here(mx);
    } else if constexpr (UNIT == 4) {
      // the scale is positive, so it commutes with the maximum
      float const m = max_across_halves(mx) * scale_log2;
      // The reference point of the exponentials moves only when the maximum has grown by more
      // than kLazy (in log2 units): until then probabilities may exceed 1 (by at most 2^kLazy,
      // harmless in fp32 sums and in bf16's range) and the running sums keep their scale, which
      // saves the rescaling of the output accumulators in nearly every tile.
      // m_new is finite: key 0 is visible to every query and tile 0 comes first.
      m_new = m > m_run + kLazy ? m : m_run;
      alpha = __builtin_amdgcn_exp2f(m_run - m_new);
      sum = 0.0f;
      here(m_new);
      here(alpha);
    } else {
      constexpr int first = (UNIT - 5) * 3;
      constexpr int last = first + 3 < 32 ? first + 3 : 32;
#pragma unroll
      for (int e = first; e < last; e++) {
        float const x = __builtin_amdgcn_exp2f(__builtin_fmaf(s[e / 16][e % 16], scale_log2, -m_new));
        pv[e / 16][e % 16] = x;
        sum += x;
        here(pv[e / 16][e % 16]);
      }
      here(sum);
    }
  }
  // probabilities as B-operand fragments; updates the running maximum and this lane's share of the sum
  __device__ __forceinline__ void finish(bf16x8 (&pf)[4], float &m_run, float &l_part) {
#pragma unroll
    for (int j = 0; j < 2; j++) {
      pf[2 * j] = pack8(pv[j]);
      pf[2 * j + 1] = pack8(pv[j] + 8);
    }
    l_part = l_part * alpha + sum;
    m_run = m_new;
  }
};

template <int D>
__global__ __launch_bounds__(256) void attn_fwd_wide_kernel(AttnParams p) {
  using C = AttnFwdCfg<D>;
  __shared__ __attribute__((aligned(1024))) bf16 Ks[2][C::kTileElems];
  __shared__ __attribute__((aligned(1024))) bf16 Vs[2][C::kTileElems];
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
  int const wq0 = q0 + wave * 64;  // first query row of this wave
  int qrow[2];
  qrow[0] = wq0 + (lane & 31);
  qrow[1] = qrow[0] + 32;
  bf16 const *qp = p.q + (int64_t)b * p.q_bs + (int64_t)head * D;
  bf16 const *kp = p.k + (int64_t)b * p.k_bs + (int64_t)head * D;
  bf16 const *vp = p.v + (int64_t)b * p.v_bs + (int64_t)head * D;

  // Q as the B operand of S^T = K Q^T: column = query row, k = d.
  bf16x8 qf[2][D / 16];
#pragma unroll
  for (int c = 0; c < 2; c++) {
    int const r = min(qrow[c], p.Sq - 1);
#pragma unroll
    for (int kk = 0; kk < D / 16; kk++) {
      qf[c][kk] = *reinterpret_cast<bf16x8 const *>(qp + (int64_t)r * p.q_ss + kk * 16 + h32 * 8);
    }
  }

  int kv_end = p.Skv;
  if (p.causal) kv_end = min(p.Skv, q0 + C::kBQ);
  int const ntiles = (kv_end + C::kBKV - 1) / C::kBKV;

  // Direct loads of a K/V tile: thread slot c (of 256 per load) writes LDS chunk c of the load's
  // 4 KB; it fetches the chunk that the swizzle puts there.  The lane's byte offsets inside the
  // tile never change; the tile and the load number move a scalar base.
  int const slot_row = t / C::kCPR, slot_pc = t % C::kCPR;
  int const k_lc = slot_pc ^ C::kswz(slot_row);
  int const v_lc = ((((slot_pc >> 2) ^ C::vswz(slot_row)) << 2) | (slot_pc & 3));
  unsigned const ks_addr = lds_address_of(&Ks[0][0]), vs_addr = lds_address_of(&Vs[0][0]);
  // byte offsets of this lane's 2 * kLoads chunks inside a tile that lies wholly below Skv
  unsigned k_voff[C::kLoads], v_voff[C::kLoads];
#pragma unroll
  for (int i = 0; i < C::kLoads; i++) {
    k_voff[i] = (unsigned)((slot_row + i * C::kRowsPerLoad) * p.k_ss + k_lc * 8) * 2u;
    v_voff[i] = (unsigned)((slot_row + i * C::kRowsPerLoad) * p.v_ss + v_lc * 8) * 2u;
  }
  // The 2 * kLoads loads of the tile at kv0 (K's, then V's) into buffer buf.  One wavefront per
  // SIMD issues one instruction every four cycles whatever its kind, so what surrounds the loads
  // counts: a tile wholly below Skv (all but the last) takes two descriptors and, per load, the
  // LDS address, M0 and the load; the row clamp of the last tile sits behind one branch per tile.
  // (Placing the loads one by one between the MFMAs of phases 1 and 2 instead of issuing them
  // together at the top of the tile was measured 10% slower.)
  auto issue_tile = [&](int kv0, int buf) {
    i32x4 const k_rsrc = buffer_resource(kp + (int64_t)kv0 * p.k_ss);
    i32x4 const v_rsrc = buffer_resource(vp + (int64_t)kv0 * p.v_ss);
    unsigned const k_dst = ks_addr + (unsigned)(buf * C::kTileElems * 2 + wave * 1024);
    unsigned const v_dst = vs_addr + (unsigned)(buf * C::kTileElems * 2 + wave * 1024);
    if (kv0 + C::kBKV > p.Skv) {  // uniform
      // rows past the last key repeat it (their scores are masked, their probabilities 0)
#pragma unroll
      for (int i = 0; i < C::kLoads; i++) {
        int const r = min(slot_row + i * C::kRowsPerLoad, p.Skv - 1 - kv0);
        lds_dma16(k_rsrc, (unsigned)(r * p.k_ss + k_lc * 8) * 2u, 0u, k_dst + (unsigned)(i * 4096));
      }
#pragma unroll
      for (int i = 0; i < C::kLoads; i++) {
        int const r = min(slot_row + i * C::kRowsPerLoad, p.Skv - 1 - kv0);
        lds_dma16(v_rsrc, (unsigned)(r * p.v_ss + v_lc * 8) * 2u, 0u, v_dst + (unsigned)(i * 4096));
      }
    } else {
#pragma unroll
      for (int i = 0; i < C::kLoads; i++) lds_dma16(k_rsrc, k_voff[i], 0u, k_dst + (unsigned)(i * 4096));
#pragma unroll
      for (int i = 0; i < C::kLoads; i++) lds_dma16(v_rsrc, v_voff[i], 0u, v_dst + (unsigned)(i * 4096));
    }
  };

  f32x16 oacc[2][D / 32];
#pragma unroll
  for (int c = 0; c < 2; c++)
#pragma unroll
    for (int i = 0; i < D / 32; i++)
#pragma unroll
      for (int r = 0; r < 16; r++) oacc[c][i][r] = 0.0f;
  float m_run[2] = {-INFINITY, -INFINITY};
  float l_part[2] = {0.0f, 0.0f};  // this lane's 16 of every 32 keys; the two lane halves meet at the end

  // Fragment addresses: everything lane-dependent is tabulated here.
  // K fragment (key block j, d step kk): row j*32 + l%32, chunk (2 kk + l/32) ^ kswz(row).
  int k_off[D / 16];
#pragma unroll
  for (int kk = 0; kk < D / 16; kk++) {
    k_off[kk] = (lane & 31) * D + (((2 * kk + h32) ^ C::kswz(lane & 31)) << 3);
  }
  // V fragment (d block i): rows 4 (l/32) + (l%16)/4 (+ 8) of a 16-row step, 4 columns at
  // 16 ((l/16)%2) + 4 (l%4) of segment i ^ vswz(row); the steps' rows are multiples of 4.
  int v_off[D / 32];
  {
    int const i16 = lane & 15;
    int const lr = 4 * h32 + (i16 >> 2);
#pragma unroll
    for (int i = 0; i < D / 32; i++) {
      v_off[i] = lr * D + ((i ^ C::vswz(lr)) << 5) + ((lane >> 4) & 1) * 16 + (i16 & 3) * 4;
    }
  }
  auto k_frag = [&](bf16 const *tile, int j, int kk) -> bf16x8 {
    return *reinterpret_cast<bf16x8 const *>(tile + k_off[kk] + j * 32 * D);
  };
  auto v_frag = [&](bf16 const *tile, int js, int i) -> bf16x8 {
    bf16 const *q = tile + v_off[i] + js * 16 * D;  // js = 2 (key block) + step
    s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(q));
    s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(q + 8 * D));
    union {
      s16x4 h2[2];
      bf16x8 v;
    } u;
    u.h2[0] = lo;
    u.h2[1] = hi;
    return u.v;
  };
  issue_tile(0, 0);
  wait_all_vmem_known_to_compiler();  // the Q fragments too: no wait for them inside the loop
  __syncthreads();
  // One tile.  The buffer index is a compile-time constant (the loop below takes tiles in
  // pairs), so that it reaches the LDS reads as an immediate offset and not through vector
  // address arithmetic per fragment: a wave alone on its SIMD pays four cycles for every
  // instruction it issues.
  auto tile_step = [&](int it, auto buffer_tag) __attribute__((always_inline)) {
    constexpr int cur = decltype(buffer_tag)::value;
    int const kv0 = it * C::kBKV;
    bool const more = it + 1 < ntiles;
    // the buffer that tile it-1 was read from is free since the barrier that ended that tile
    if (more) issue_tile(kv0 + C::kBKV, cur ^ 1);

    // A wave whose rows all lie before this tile (causal) has nothing to add.  A half whose rows
    // all do is computed with every score masked, which leaves its state as it is.
    bool const active = !p.causal || kv0 <= wq0 + 63;
    if (active) {
      bf16 const *kt = Ks[cur];
      bf16 const *vt = Vs[cur];
      // wave-uniform: may an element of this tile need masking (end of the keys, causal diagonal)?
      bool const edge = (kv0 + C::kBKV > p.Skv) || (p.causal && kv0 + C::kBKV - 1 > wq0);
      auto mask = [&](f32x16 (&s)[2], int c) {
#pragma unroll
        for (int j = 0; j < 2; j++) {
#pragma unroll
          for (int r = 0; r < 16; r++) {
            int const kv = kv0 + j * 32 + 8 * (r >> 2) + 4 * h32 + (r & 3);
            if (kv >= p.Skv || (p.causal && kv > qrow[c])) s[j][r] = -INFINITY;
          }
        }
      };
      auto rescale = [&](int c, float alpha) {
        // only when some row's maximum moved
        if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
          asm volatile("" ::: "memory");  // keeps the multiplications under the branch
#pragma unroll
          for (int i = 0; i < D / 32; i++)
#pragma unroll
            for (int r = 0; r < 16; r++) oacc[c][i][r] *= alpha;
        }
      };

      // ---- phase 1: K fragments, S_0^T (rows = keys, columns = this half's queries) ----
      bf16x8 kf[2][D / 16];
#pragma unroll
      for (int kk = 0; kk < D / 16; kk++)
#pragma unroll
        for (int j = 0; j < 2; j++) kf[j][kk] = k_frag(kt, j, kk);
      f32x16 s0[2], s1[2];
#pragma unroll
      for (int j = 0; j < 2; j++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
          s0[j][r] = 0.0f;
          s1[j][r] = 0.0f;
        }
      // the two key blocks alternate, so that no MFMA waits for the one just before it
      constexpr int NM = D / 8;               // MFMAs of a phase
      static_for<0, NM>([&](auto mc) {
        constexpr int m = decltype(mc)::value;
        constexpr int kk = m / 2, j = m % 2;
        __builtin_amdgcn_sched_barrier(0);
        s0[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[j][kk], qf[0][kk], s0[j], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      });
      __builtin_amdgcn_sched_barrier(0);
      if (edge) mask(s0, 0);

      // ---- phase 2: S_1^T on the matrix pipe, softmax of S_0 on the vector ALU ----
      // One MFMA, then one or two units of the softmax, fenced so that the order stays as written:
      // the wave issues the vector instructions while the matrix pipe works on the MFMA.
      constexpr int UPM = 16 / NM;        // softmax units behind each MFMA
      bf16x8 pf0[4], pf1[4];
      SoftmaxHalf sm;
      static_for<0, NM>([&](auto mc) {
        constexpr int m = decltype(mc)::value;
        constexpr int kk = m / 2, j = m % 2;
        __builtin_amdgcn_sched_barrier(0);
        s1[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[j][kk], qf[1][kk], s1[j], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        static_for<0, UPM>([&](auto uc) { sm.template unit<m * UPM + decltype(uc)::value>(s0, p.scale_log2, m_run[0]); });
      });
      __builtin_amdgcn_sched_barrier(0);
      float const alpha0 = sm.alpha;
      sm.finish(pf0, m_run[0], l_part[0]);
      rescale(0, alpha0);
      if (edge) mask(s1, 1);

      // ---- phase 3: V fragments, O_0^T += V^T P_0^T; softmax of S_1 ----
      // A = V^T (rows d) via transposing loads, B = P^T; (key block, step) outside, d blocks inside.
      // The fragment of an MFMA is read kAhead slots ahead of it (an LDS read takes longer than
      // one MFMA, more so while the direct loads write into the other buffer).
      constexpr int kAhead = 3;
      bf16x8 vf[D / 32][4];
#pragma unroll
      for (int m = 0; m < kAhead; m++) vf[m % (D / 32)][m / (D / 32)] = v_frag(vt, m / (D / 32), m % (D / 32));
      static_for<0, NM>([&](auto mc) {
        constexpr int m = decltype(mc)::value;
        constexpr int js = m / (D / 32), i = m % (D / 32);
        __builtin_amdgcn_sched_barrier(0);
        oacc[0][i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[i][js], pf0[js], oacc[0][i], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (m + kAhead < NM) {
          constexpr int js1 = (m + kAhead) / (D / 32), i1 = (m + kAhead) % (D / 32);
          vf[i1][js1] = v_frag(vt, js1, i1);
        }
        static_for<0, UPM>([&](auto uc) { sm.template unit<m * UPM + decltype(uc)::value>(s1, p.scale_log2, m_run[1]); });
      });
      __builtin_amdgcn_sched_barrier(0);
      float const alpha1 = sm.alpha;
      sm.finish(pf1, m_run[1], l_part[1]);
      rescale(1, alpha1);

      // ---- phase 4: O_1^T += V^T P_1^T with the fragments still in registers ----
#pragma unroll
      for (int js = 0; js < 4; js++)
#pragma unroll
        for (int i = 0; i < D / 32; i++)
          oacc[1][i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[i][js], pf1[js], oacc[1][i], 0, 0, 0);
    }
    wait_vmcnt<0>();  // this wave's part of the next tile has landed
    __syncthreads();
  };
  for (int it = 0; it < ntiles; it += 2) {
    tile_step(it, std::integral_constant<int, 0>{});
    if (it + 1 < ntiles) tile_step(it + 1, std::integral_constant<int, 1>{});
  }

#pragma unroll
  for (int c = 0; c < 2; c++) {
    float const l_run = l_part[c] + __shfl_xor(l_part[c], 32, 64);
    if (qrow[c] < p.Sq) {
      float const inv = 1.0f / l_run;
      bf16 *op = p.o + (int64_t)b * p.o_bs + (int64_t)qrow[c] * p.o_ss + (int64_t)head * D;
#pragma unroll
      for (int i = 0; i < D / 32; i++) {
#pragma unroll
        for (int g = 0; g < 4; g++) {
          int d = i * 32 + 8 * g + 4 * h32;
          u32x2 w = {pack_bf16x2(oacc[c][i][4 * g] * inv, oacc[c][i][4 * g + 1] * inv),
                     pack_bf16x2(oacc[c][i][4 * g + 2] * inv, oacc[c][i][4 * g + 3] * inv)};
          *reinterpret_cast<u32x2 *>(op + d) = w;
        }
      }
      if (h32 == 0 && p.lse != nullptr) {
        p.lse[((int64_t)b * p.H + head) * p.Sq + qrow[c]] = (m_run[c] + __log2f(l_run)) * kLn2;
      }
    }
  }
}

// Launches the forward kernel for head_dim 64 or 128 (checked by the caller).
hipError_t attention_bf16_forward_wide(hipStream_t st, AttnParams const &p, int head_dim) {
  dim3 grid((unsigned)(ceil_div(p.Sq, 256) * p.H * p.B));
  if (head_dim == 64) {
    attn_fwd_wide_kernel<64><<<grid, 256, 0, st>>>(p);
  } else {
    attn_fwd_wide_kernel<128><<<grid, 256, 0, st>>>(p);
  }
  return hipGetLastError();
}

}  // namespace ffk
