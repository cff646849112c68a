// bf16 attention backward: dK/dV kernel and dQ kernel with streamed tiles
// fetched by direct global -> LDS loads.
//
// Both kernels own 128 rows per workgroup (32 per wavefront) of the tensors
// whose gradient they produce, keep those rows' operand fragments and the
// gradient accumulators in registers, and stream the other side in tiles of 64
// rows through three LDS buffers.  A tile arrives by direct loads (no register
// staging, no LDS write instructions).  One wavefront runs per SIMD, so the
// wavefront itself overlaps its matrix and vector work: a tile is two halves of
// 32 rows, and the vector work of one half (exponentials, dS) is cut into units
// that sit behind the MFMAs of the other half, in an order fenced against the
// compiler's scheduler; LDS fragments are read a few MFMAs ahead of their use.
//
// A tile lies in LDS as in memory, [32 rows][D] without padding, with the
// 16-byte chunks of a row permuted on the fetching side.  It is read in two
// ways: with 16-byte loads (rows = MFMA rows, 16 lanes = 16 rows per cycle) and
// with transposing 8-byte loads (32 lanes = 4 rows x 64 bytes per cycle).  The
// permutation chunk ^ swz(row) keeps both free of bank conflicts:
//   D = 128 (16 chunks per row):  swz(row) = (row % 4) * 4 + (row / 4) % 4
//   D = 64  (8 chunks, 2 rows per 256 bytes), x = row / 2:
//                                 swz(row) = (x % 2) * 4 + (x / 2) % 4
// Layouts of the MFMA 32x32x16 bf16 (l = lane): A operand row l%32,
// k = 8*(l/32)..+7; B operand column l%32, same k; accumulator element r:
// row 8*(r/4) + 4*(l/32) + r%4, column l%32.  An accumulator tile re-used as an
// operand takes its 8 values r = 8s..8s+7 as the k-slots of step s; the other
// operand is read with the same permutation of the reduction index by the
// transposing loads.
#include "attention_common.h"
#include "lds_dma.h"
#include <type_traits>

namespace ffk {

template <int D>
struct AttnBwd2Cfg {
  static constexpr int kBlk = 128;   // rows owned by a workgroup
  static constexpr int kTile = 64;   // rows of the streamed tensors per step: two halves of 32
  static constexpr int kCPR = D / 8;                  // 16-byte chunks per row
  static constexpr int kLoads = kTile * kCPR / 256;   // direct loads per thread, per tensor and tile
  static constexpr int kRowsPerLoad = 256 / kCPR;
  static constexpr int kTileElems = kTile * D;
  static_assert(D == 64 || D == 128, "swizzles are written for these two");
  __device__ static int swz(int row) {
    return D == 128 ? (((row & 3) << 2) | ((row >> 2) & 3)) : ((((row >> 1) & 1) << 2) | ((row >> 2) & 3));
  }
};

// Per-lane LDS offsets (in elements) of the two ways a streamed tile is read.
template <int D>
struct TileReader {
  using C = AttnBwd2Cfg<D>;
  int row_off[D / 16];      // 16-byte read of d step kk: row l%32, chunk (2 kk + l/32) ^ swz(row)
  int tr_off[D / 32][2];    // transposing read of d block i, first / second 8 rows of a 16-row step
  __device__ void init(int lane) {
    int const h32 = lane >> 5, r = lane & 31;
#pragma unroll
    for (int kk = 0; kk < D / 16; kk++) row_off[kk] = r * D + (((2 * kk + h32) ^ C::swz(r)) << 3);
    // rows 16 s + 8 sec + 4 (l/32) + (l%16)/4, 4 columns at 16 ((l/16)%2) + 4 (l%4) of block i
    int const i16 = lane & 15, q = i16 >> 2, b = (lane >> 4) & 1, c = i16 & 3;
#pragma unroll
    for (int i = 0; i < D / 32; i++) {
#pragma unroll
      for (int sec = 0; sec < 2; sec++) {
        int const row = 8 * sec + 4 * h32 + q;  // the step's 16 rows add a multiple of 16: swz ignores it
        int const chunk = 4 * i + 2 * b + (c >> 1);
        tr_off[i][sec] = row * D + ((chunk ^ C::swz(row)) << 3) + 4 * (c & 1);
      }
    }
  }
  // `tile` points at the first of the 32 rows that are read
  __device__ bf16x8 rows(bf16 const *tile, int kk) const {
    return *reinterpret_cast<bf16x8 const *>(tile + row_off[kk]);
  }
  __device__ bf16x8 transposed(bf16 const *tile, int s, int i) const {
    s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(tile + tr_off[i][0] + 16 * s * D));
    s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(tile + tr_off[i][1] + 16 * s * D));
    union {
      s16x4 h2[2];
      bf16x8 v;
    } u;
    u.h2[0] = lo;
    u.h2[1] = hi;
    return u.v;
  }
};

// (A) dK, dV: workgroup owns 128 key rows (32 per wave), streams query tiles.
template <int D>
__global__ __launch_bounds__(256) void attn_bwd_dkdv2_kernel(AttnBwdParams p) {
  using C = AttnBwd2Cfg<D>;
  constexpr int NBUF = 3;  // the tile in use and the two after it
  __shared__ __attribute__((aligned(1024))) bf16 Qs[NBUF][C::kTileElems];
  __shared__ __attribute__((aligned(1024))) bf16 Gs[NBUF][C::kTileElems];  // dO
  __shared__ __attribute__((aligned(256))) float Ls[NBUF][64], Ds[NBUF][64];  // log-sum-exp, delta of a tile's rows
  __shared__ __attribute__((aligned(256))) float Unused[64];
  int const t = threadIdx.x, lane = t & 63, h32 = lane >> 5;
  // the wave index as a scalar: tile-level decisions taken from it are branches, not lane masks
  int const wave = __builtin_amdgcn_readfirstlane(t >> 6);
  // key block 0 sees every query under a causal mask: heaviest first for all heads
  int const hb = blockIdx.x % (p.H * p.B);
  int const head = hb % p.H, b = hb / p.H;
  int const kv0 = (blockIdx.x / (p.H * p.B)) * C::kBlk;
  int const kvrow = kv0 + wave * 32 + (lane & 31);
  bf16 const *qp = p.q + (int64_t)b * p.q_bs + (int64_t)head * D;
  bf16 const *gp = p.d_o + (int64_t)b * p.o_bs + (int64_t)head * D;
  bf16 const *kp = p.k + (int64_t)b * p.k_bs + (int64_t)head * D;
  bf16 const *vp = p.v + (int64_t)b * p.v_bs + (int64_t)head * D;
  float const *lsep = p.lse + ((int64_t)b * p.H + head) * p.Sq;
  float const *delp = p.delta + ((int64_t)b * p.H + head) * p.Sq;

  // K and V rows of this lane as B operands (column = key row, k = d).
  bf16x8 kf[D / 16], vf[D / 16];
  {
    int const r = min(kvrow, p.Skv - 1);
#pragma unroll
    for (int kk = 0; kk < D / 16; kk++) {
      kf[kk] = *reinterpret_cast<bf16x8 const *>(kp + (int64_t)r * p.k_ss + kk * 16 + h32 * 8);
      vf[kk] = *reinterpret_cast<bf16x8 const *>(vp + (int64_t)r * p.v_ss + kk * 16 + h32 * 8);
    }
  }
  f32x16 dk[D / 32], dv[D / 32];
#pragma unroll
  for (int i = 0; i < D / 32; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) {
      dk[i][r] = 0.0f;
      dv[i][r] = 0.0f;
    }

  int const q_begin = p.causal ? (kv0 / C::kTile) * C::kTile : 0;
  int const ntiles = (p.Sq - q_begin + C::kTile - 1) / C::kTile;

  // Direct loads of a tile: thread slot c (of 256 per load) writes LDS chunk c of the load's 4 KB
  // and fetches the chunk that the permutation puts there.  Rows past the last query repeat it
  // (what is computed from them is masked).  Waves 0 and 1 also fetch the tile's 64 log-sum-exp
  // and delta values.
  int const slot_row = t / C::kCPR, slot_lc = (t % C::kCPR) ^ C::swz(t / C::kCPR);
  unsigned const qs_addr = lds_address_of(&Qs[0][0]), gs_addr = lds_address_of(&Gs[0][0]);
  unsigned const ls_addr = lds_address_of(&Ls[0][0]), ds_addr = lds_address_of(&Ds[0][0]);
  // One descriptor per tensor for the whole kernel; the tile moves a scalar byte offset (the host
  // has checked that a (batch, head)'s rows span less than 4 GB).  Every wave issues the same
  // number of loads per tile (waves 2 and 3 fetch the log-sum-exp / delta values a second time,
  // into 256 bytes nobody reads), so that one wait count fits all.
  i32x4 const rq = buffer_resource(qp), rg = buffer_resource(gp);
  i32x4 const rs = buffer_resource((wave & 1) == 0 ? lsep : delp);
  unsigned const unused_addr = lds_address_of(&Unused[0]);
  constexpr int kLoadsPerTile = 2 * C::kLoads + 1;
  // (Issuing these loads one by one between the MFMAs of the phases without vector work, instead
  // of together at the top of the step, was measured 6% slower.)
  auto issue_tile = [&](int qt0, int buf) {
    int const last = p.Sq - 1 - qt0;  // >= 0 for every tile that is used
    unsigned const q_tile = (unsigned)qt0 * (unsigned)p.q_ss * 2u, g_tile = (unsigned)qt0 * (unsigned)p.o_ss * 2u;
#pragma unroll
    for (int i = 0; i < C::kLoads; i++) {
      int const r = min(slot_row + i * C::kRowsPerLoad, last);
      unsigned const dst = (unsigned)(buf * C::kTileElems * 2 + (i * 4 + wave) * 1024);
      lds_dma16(rq, (unsigned)(r * p.q_ss + slot_lc * 8) * 2u, q_tile, qs_addr + dst);
      lds_dma16(rg, (unsigned)(r * p.o_ss + slot_lc * 8) * 2u, g_tile, gs_addr + dst);
    }
    lds_dma4(rs, (unsigned)min(lane, last) * 4u, (unsigned)qt0 * 4u,
             wave >= 2 ? unused_addr : (wave == 0 ? ls_addr : ds_addr) + (unsigned)buf * 256u);
  };

  TileReader<D> rd;
  rd.init(lane);
  // Tiles past the end are fetched too while they start below Sq (their rows repeat the last
  // one); nothing is done with them.
  // Tile it+2 is fetched during step it (a fetch takes longer than one step while eight waves
  // per CU stream tiles).  A fetch is issued for every step, past the end the last tile again
  // into a buffer nobody reads any more: the count of loads in flight is then the same at every
  // wait.
  int const last_tile = q_begin + (ntiles - 1) * C::kTile;
  if (ntiles > 0) {
    issue_tile(q_begin, 0);
    issue_tile(min(q_begin + C::kTile, last_tile), 1);
  }
  // Tiles 0 and 1 have landed, and so have the K and V fragments: told to the compiler, which
  // otherwise waits for those fragments at their uses in every step, where the counter holds the
  // two tiles in flight.
  wait_all_vmem_known_to_compiler();
  __syncthreads();
  int cur = 0;
  for (int it = 0; it < ntiles; it++) {
    int const qt0 = q_begin + it * C::kTile;
    // buffer (it+2) % 3 was read during step it-1; every wave has passed the barrier that ended it
    issue_tile(min(qt0 + 2 * C::kTile, last_tile), cur == 0 ? 2 : cur - 1);
    // A wave whose keys all lie after this query tile (causal) contributes 0.  A half whose
    // queries all lie before the wave's keys is computed with everything masked: it adds zeros.
    bool const active = !p.causal || kv0 + wave * 32 <= qt0 + C::kTile - 1;
    if (active) {
      bf16 const *qt = Qs[cur], *gt = Gs[cur];
      // wave-uniform: does any element of this wave's 64 x 32 block need masking?
      bool const edge = qt0 + C::kTile > p.Sq || kv0 + wave * 32 + 32 > p.Skv || (p.causal && kv0 + wave * 32 + 31 > qt0);
      constexpr int NM = D / 8;       // MFMAs of a phase
      constexpr int UPM = 16 / NM;    // units of vector work behind each
      constexpr int kAhead = 3;       // an LDS fragment is read this many MFMAs ahead of its use
      constexpr int NI = D / 32;
      // S = Q K^T and dP = dO V^T of one half: rows = its 32 queries, column = key.  MFMA m takes
      // fragment m: d step m / 2 of Q (m even, into S) or of dO (m odd, into dP).
      auto sdp_frag = [&](int h, int m) __attribute__((always_inline)) {
        return rd.rows(((m & 1) ? gt : qt) + h * 32 * D, m >> 1);
      };
      // dV += P^T dO ; dK += dS^T Q of one half.  A = the probabilities / dS re-used from the
      // accumulator layout (row = key), B = dO / Q read with the matching reduction order
      // (k = query).  MFMA m: step s2 = m / (2 NI), d block (m / 2) % NI, dO (m even) or Q.
      auto grad_frag = [&](int h, int m) __attribute__((always_inline)) {
        return rd.transposed(((m & 1) ? qt : gt) + h * 32 * D, m / (2 * NI), (m >> 1) % NI);
      };
      // The vector work of a half, 16 units of one score each: P = exp(S scale - lse),
      // dS = P (dP - delta) scale.  Unit 4 g reads the statistics of rows 8 g + 4 (l/32) .. + 3.
      float pv[2][16], dsv[2][16];
      f32x4 lrow, drow;
      auto unit = [&](int h, int u, f32x16 const &s, f32x16 const &dp) __attribute__((always_inline)) {
        if ((u & 3) == 0) {
          lrow = *reinterpret_cast<f32x4 const *>(&Ls[cur][h * 32 + 2 * u + 4 * h32]);
          drow = *reinterpret_cast<f32x4 const *>(&Ds[cur][h * 32 + 2 * u + 4 * h32]);
        }
        float const e = __builtin_amdgcn_exp2f(__builtin_fmaf(s[u], p.scale_log2, -(lrow[u & 3] * kLog2e)));
        pv[h][u] = e;
        dsv[h][u] = e * __builtin_fmaf(dp[u], p.scale, -(drow[u & 3] * p.scale));
        pin_here(pv[h][u]);
        pin_here(dsv[h][u]);
      };
      auto mask_half = [&](int h) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
          int const qg = qt0 + h * 32 + 8 * (r >> 2) + 4 * h32 + (r & 3);
          bool const masked = qg >= p.Sq || kvrow >= p.Skv || (p.causal && kvrow > qg);
          pv[h][r] = masked ? 0.0f : pv[h][r];
          dsv[h][r] = masked ? 0.0f : dsv[h][r];
        }
      };
      f32x16 s[2], dp[2];
#pragma unroll
      for (int h = 0; h < 2; h++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
          s[h][r] = 0.0f;
          dp[h][r] = 0.0f;
        }
      bf16x8 fr[NM];

      // ---- phase 1: S, dP of half 0 ----
#pragma unroll
      for (int m = 0; m < kAhead; m++) fr[m] = sdp_frag(0, m);
      static_for<0, NM>([&](auto mc) {
        constexpr int m = decltype(mc)::value;
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (m % 2 == 0) {
          s[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fr[m], kf[m / 2], s[0], 0, 0, 0);
        } else {
          dp[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fr[m], vf[m / 2], dp[0], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (m + kAhead < NM) fr[m + kAhead] = sdp_frag(0, m + kAhead);
      });
      __builtin_amdgcn_sched_barrier(0);

      // ---- phase 2: S, dP of half 1 on the matrix pipe, P and dS of half 0 on the vector ALU ----
      bf16x8 fr2[NM];
#pragma unroll
      for (int m = 0; m < kAhead; m++) fr2[m] = sdp_frag(1, m);
      static_for<0, NM>([&](auto mc) {
        constexpr int m = decltype(mc)::value;
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (m % 2 == 0) {
          s[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fr2[m], kf[m / 2], s[1], 0, 0, 0);
        } else {
          dp[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fr2[m], vf[m / 2], dp[1], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (m + kAhead < NM) fr2[m + kAhead] = sdp_frag(1, m + kAhead);
        static_for<0, UPM>([&](auto uc) { unit(0, m * UPM + decltype(uc)::value, s[0], dp[0]); });
      });
      __builtin_amdgcn_sched_barrier(0);
      if (edge) mask_half(0);
      bf16x8 pa[2][2], da[2][2];
#pragma unroll
      for (int s2 = 0; s2 < 2; s2++) {
        pa[0][s2] = pack8(pv[0] + 8 * s2);
        da[0][s2] = pack8(dsv[0] + 8 * s2);
      }

      // ---- phase 3: dV, dK of half 0 on the matrix pipe, P and dS of half 1 on the vector ALU ----
      bf16x8 fr3[NM];
#pragma unroll
      for (int m = 0; m < kAhead; m++) fr3[m] = grad_frag(0, m);
      static_for<0, NM>([&](auto mc) {
        constexpr int m = decltype(mc)::value;
        constexpr int s2 = m / (2 * NI), i = (m / 2) % NI;
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (m % 2 == 0) {
          dv[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(pa[0][s2], fr3[m], dv[i], 0, 0, 0);
        } else {
          dk[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(da[0][s2], fr3[m], dk[i], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (m + kAhead < NM) fr3[m + kAhead] = grad_frag(0, m + kAhead);
        static_for<0, UPM>([&](auto uc) { unit(1, m * UPM + decltype(uc)::value, s[1], dp[1]); });
      });
      __builtin_amdgcn_sched_barrier(0);
      if (edge) mask_half(1);
#pragma unroll
      for (int s2 = 0; s2 < 2; s2++) {
        pa[1][s2] = pack8(pv[1] + 8 * s2);
        da[1][s2] = pack8(dsv[1] + 8 * s2);
      }

      // ---- phase 4: dV, dK of half 1 ----
      bf16x8 fr4[NM];
#pragma unroll
      for (int m = 0; m < kAhead; m++) fr4[m] = grad_frag(1, m);
      static_for<0, NM>([&](auto mc) {
        constexpr int m = decltype(mc)::value;
        constexpr int s2 = m / (2 * NI), i = (m / 2) % NI;
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (m % 2 == 0) {
          dv[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(pa[1][s2], fr4[m], dv[i], 0, 0, 0);
        } else {
          dk[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(da[1][s2], fr4[m], dk[i], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (m + kAhead < NM) fr4[m + kAhead] = grad_frag(1, m + kAhead);
      });
      __builtin_amdgcn_sched_barrier(0);
    }
    wait_vmcnt<kLoadsPerTile>();  // this wave's part of the next tile has landed
    __syncthreads();
    cur = cur == 2 ? 0 : cur + 1;
  }
  wait_vmcnt<0>();
  __syncthreads();  // the buffers are free: no load is in flight, no wave reads a tile

  // dK / dV accumulators: row = key (32 per wave, 8*(r/4)+4*h+r%4), column = d: a lane
  // holds one column of 16 rows.  Each wave turns its 32 x D block around in LDS (the
  // streamed tiles are done with) and writes whole 16-byte pieces of rows.
  constexpr int kOutStride = D;  // a wave writes rows of 32 consecutive columns and reads whole rows: no padding needed
  bf16 *const stage = (wave < 2 ? &Qs[0][0] : &Gs[0][0]) + (wave & 1) * 32 * kOutStride;
  static_assert(2 * 32 * kOutStride <= NBUF * C::kTileElems, "staging fits the tile buffers");
  auto write_out = [&](f32x16 const (&acc)[D / 32], bf16 *out, int64_t row_stride) {
#pragma unroll
    for (int i = 0; i < D / 32; i++) {
#pragma unroll
      for (int r = 0; r < 16; r++) {
        int const row = 8 * (r >> 2) + 4 * h32 + (r & 3);
        VecIO<bf16>::store1(stage + row * kOutStride + i * 32 + (lane & 31), acc[i][r]);
      }
    }
    // LDS operations of one wave complete in order: the reads below see the writes above
#pragma unroll
    for (int k = 0; k < 32 * (D / 8) / 64; k++) {
      int const c = lane + k * 64;
      int const row = c / (D / 8), ch = c % (D / 8);
      u32x4 const v = *reinterpret_cast<u32x4 const *>(stage + row * kOutStride + ch * 8);
      int const grow = kv0 + wave * 32 + row;
      if (grow < p.Skv) *reinterpret_cast<u32x4 *>(out + (int64_t)grow * row_stride + ch * 8) = v;
    }
  };
  write_out(dk, p.dk + (int64_t)b * p.k_bs + (int64_t)head * D, p.k_ss);
  write_out(dv, p.dv + (int64_t)b * p.v_bs + (int64_t)head * D, p.v_ss);
}

// Whether the kernels of this file can address the problem: a tile's byte offset inside a
// (batch, head)'s rows is a 32-bit scalar.
hipError_t attention_bf16_dkdv(hipStream_t st, AttnBwdParams const &p, int head_dim) {
  dim3 grid((unsigned)(ceil_div(p.Skv, 128) * p.H * p.B));
  if (head_dim == 64) {
    attn_bwd_dkdv2_kernel<64><<<grid, 256, 0, st>>>(p);
  } else {
    attn_bwd_dkdv2_kernel<128><<<grid, 256, 0, st>>>(p);
  }
  return hipGetLastError();
}

}  // namespace ffk
