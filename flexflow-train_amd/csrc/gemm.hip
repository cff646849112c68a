// GEMM kernels for gfx950 behind Linear and the attention projections.
//
//  * bf16: LDS-tiled, double-buffered MFMA kernel (v_mfma_f32_32x32x16_bf16,
//    fp32 accumulators, one rounding at the store).  Operands whose reduction
//    dimension is not contiguous in memory are staged into LDS as they lie in
//    memory and read back with the transposing LDS load (ds_read_b64_tr_b16),
//    so all four transpose variants run on the same pipeline.
//  * fp32: MFMA v_mfma_f32_32x32x2f32 kernel with bounds-checked loads, used
//    for the fp32 Linear (small, latency-bound shapes).
//  * a plain one-thread-per-output kernel for shapes the tiled bf16 kernel
//    cannot take (K or leading dimensions not a multiple of 8 elements).
//
// These replace the cublasGemmEx calls of the reference
// (lib/kernels/src/cuda/ops/linear_kernels.cu:143,163,249,298,321).
#include "lds_dma.h"
#include "gemm.h"
#include "colreduce.h"
#include <stdarg.h>
#include <stdlib.h>
#include <type_traits>

namespace ffk {

__device__ __forceinline__ float apply_activation(float v, int act) {
  switch (act) {
    case FFK_ACT_RELU:
      // tensor_accessor_relu keeps x >= 0 (tensor_accessor_unary_ops.cc:32-38);
      // identical to x > 0 ? x : 0 on every input except -0.0f.
      return v >= 0.0f ? v : 0.0f;
    case FFK_ACT_SIGMOID:
      return 1.0f / (1.0f + expf(-v));
    case FFK_ACT_TANH:
      return tanhf(v);
    case FFK_ACT_GELU:
      return gelu_forward(v);
    default:
      return v;
  }
}

// ---------------------------------------------------------------------------
// Block -> tile mapping.  Workgroups are dealt round-robin to the 8 XCDs, each
// with its own L2; regroup ids so that one XCD works on a compact patch of the
// output (tiles that share A rows / B columns), then walk the patch in groups
// of kGroupM tile rows.
// ---------------------------------------------------------------------------
__device__ __forceinline__ void tile_coords(int pid, int nbm, int nbn, int &tm,
                                            int &tn) {
  int const total = nbm * nbn;
  if (total % kNumXCD == 0) {
    int const xcd = pid % kNumXCD;
    int const local = pid / kNumXCD;
    pid = xcd * (total / kNumXCD) + local;
  }
  constexpr int kGroupM = 8;
  int const group_size = kGroupM * nbn;
  int const group = pid / group_size;
  int const first_m = group * kGroupM;
  int const rows = min(nbm - first_m, kGroupM);
  int const in_group = pid % group_size;
  tm = first_m + in_group % rows;
  tn = in_group / rows;
}

// ---------------------------------------------------------------------------
// Asking instead of launching: while this thread's name sink is set (by
// ffk_gemm_kernel_name), every launch site below writes the kernel it would
// have launched into the sink and returns without touching the device.
// ---------------------------------------------------------------------------
static thread_local char *tl_name_sink = nullptr;
static thread_local size_t tl_name_sink_bytes = 0;
static bool describe_only(char const *fmt, ...) __attribute__((format(printf, 1, 2)));
static bool describe_only(char const *fmt, ...) {
  if (tl_name_sink == nullptr) return false;
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(tl_name_sink, tl_name_sink_bytes, fmt, ap);
  va_end(ap);
  return true;
}
static char const *tf(bool b) { return b ? "true" : "false"; }

// ---------------------------------------------------------------------------
// bf16 MFMA kernel
// ---------------------------------------------------------------------------
constexpr int kBK = 64;        // K extent of one LDS tile
constexpr int kPadK = 8;       // row padding (elements) of a K-contiguous tile
constexpr int kPadMN = 32;     // row padding of an M/N-contiguous tile

template <int ROWS, bool TRANS>
struct TileGeom {
  // TRANS == false: tile held as [ROWS][kBK] (reduction dim contiguous)
  // TRANS == true : tile held as [kBK][ROWS] (as it lies in memory)
  static constexpr int kStride = TRANS ? (ROWS + kPadMN) : (kBK + kPadK);
  static constexpr int kElems = TRANS ? kBK * kStride : ROWS * kStride;
};

template <int BM, int BN, int WM, int WN, bool TA, bool TB, bool EDGE>
__global__ __launch_bounds__((BM / WM) * (BN / WN) * 64) void gemm_bf16_kernel(
    bf16 const *__restrict__ A, bf16 const *__restrict__ B, bf16 *C, int M,
    int N, int K, int64_t lda, int64_t ldb, int64_t ldc,
    bf16 const *__restrict__ bias, int act, int accumulate) {
  constexpr int NW = (BM / WM) * (BN / WN);
  constexpr int NT = NW * 64;
  constexpr int TM = WM / 32;  // MFMA tiles per wave along M
  constexpr int TN = WN / 32;
  using GA = TileGeom<BM, TA>;
  using GB = TileGeom<BN, TB == false>;  // B is "transposed" when it is [K,N]
  constexpr bool TBL = (TB == false);    // B tile lies as [kBK][BN]
  constexpr int A_CHUNKS = BM * kBK / 8 / NT;  // 16-byte chunks per thread
  constexpr int B_CHUNKS = BN * kBK / 8 / NT;
  static_assert(BM * kBK / 8 % NT == 0 && BN * kBK / 8 % NT == 0, "tile/threads");

  __shared__ __attribute__((aligned(16))) bf16 As[2][GA::kElems];
  __shared__ __attribute__((aligned(16))) bf16 Bs[2][GB::kElems];

  int const t = threadIdx.x;
  int const lane = t & 63;
  int const wave = t >> 6;
  int const wm0 = (wave / (BN / WN)) * WM;
  int const wn0 = (wave % (BN / WN)) * WN;

  int tm, tn;
  tile_coords(blockIdx.x, (M + BM - 1) / BM, (N + BN - 1) / BN, tm, tn);
  int const m0 = tm * BM;
  int const n0 = tn * BN;

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

  u32x4 ra[A_CHUNKS], rb[B_CHUNKS];

  auto gload = [&](int k0) {
#pragma unroll
    for (int i = 0; i < A_CHUNKS; i++) {
      int c = t + i * NT;
      int64_t off;
      bool ok = true;
      if (!TA) {
        int row = c >> 3, kc = c & 7;
        int gm = m0 + row, gk = k0 + kc * 8;
        if (EDGE) {
          gm = min(gm, M - 1);
          ok = gk < K;
          gk = ok ? gk : 0;
        }
        off = (int64_t)gm * lda + gk;
      } else {
        int krow = c / (BM / 8), mc = c % (BM / 8);
        int gk = k0 + krow, gm = m0 + mc * 8;
        if (EDGE) {
          ok = gk < K && gm < M;  // M % 8 == 0 is required, so chunks are whole
          gk = ok ? gk : 0;
          gm = ok ? gm : 0;
        }
        off = (int64_t)gk * lda + gm;
      }
      u32x4 v = *reinterpret_cast<u32x4 const *>(A + off);
      if (EDGE && !ok) v = u32x4{0u, 0u, 0u, 0u};
      ra[i] = v;
    }
#pragma unroll
    for (int i = 0; i < B_CHUNKS; i++) {
      int c = t + i * NT;
      int64_t off;
      bool ok = true;
      if (!TBL) {
        int row = c >> 3, kc = c & 7;
        int gn = n0 + row, gk = k0 + kc * 8;
        if (EDGE) {
          gn = min(gn, N - 1);
          ok = gk < K;
          gk = ok ? gk : 0;
        }
        off = (int64_t)gn * ldb + gk;
      } else {
        int krow = c / (BN / 8), nc = c % (BN / 8);
        int gk = k0 + krow, gn = n0 + nc * 8;
        if (EDGE) {
          ok = gk < K && gn < N;
          gk = ok ? gk : 0;
          gn = ok ? gn : 0;
        }
        off = (int64_t)gk * ldb + gn;
      }
      u32x4 v = *reinterpret_cast<u32x4 const *>(B + off);
      if (EDGE && !ok) v = u32x4{0u, 0u, 0u, 0u};
      rb[i] = v;
    }
  };

  auto lstore = [&](int buf) {
#pragma unroll
    for (int i = 0; i < A_CHUNKS; i++) {
      int c = t + i * NT;
      int idx;
      if (!TA) {
        idx = (c >> 3) * GA::kStride + (c & 7) * 8;
      } else {
        idx = (c / (BM / 8)) * GA::kStride + (c % (BM / 8)) * 8;
      }
      *reinterpret_cast<u32x4 *>(&As[buf][idx]) = ra[i];
    }
#pragma unroll
    for (int i = 0; i < B_CHUNKS; i++) {
      int c = t + i * NT;
      int idx;
      if (!TBL) {
        idx = (c >> 3) * GB::kStride + (c & 7) * 8;
      } else {
        idx = (c / (BN / 8)) * GB::kStride + (c % (BN / 8)) * 8;
      }
      *reinterpret_cast<u32x4 *>(&Bs[buf][idx]) = rb[i];
    }
  };

  // Operand fragment for one 32-row MFMA tile and one 16-wide k step.
  // Lane l supplies row (l % 32), k = 8 * (l / 32) .. + 7.
  auto frag = [&](bf16 const *tile, int stride, bool trans, int row0,
                  int kk) -> bf16x8 {
    if (!trans) {
      bf16 const *p = tile + (row0 + (lane & 31)) * stride + kk * 16 + (lane >> 5) * 8;
      return *reinterpret_cast<bf16x8 const *>(p);
    }
    // Transposing load: within each 16-lane group, lane i points at 4 elements
    // of row k_(i/4), columns 4*(i%4)..+3, and receives column i of the four
    // rows.  Two loads give 8 consecutive k for this lane's row.
    int const i16 = lane & 15;
    int const col = row0 + ((lane >> 4) & 1) * 16 + (i16 & 3) * 4;
    int const kbase = kk * 16 + (lane >> 5) * 8 + (i16 >> 2);
    typedef s16x4 __attribute__((address_space(3))) * lds_s16x4_ptr;
    s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
        (lds_s16x4_ptr)(tile + kbase * stride + col));
    s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
        (lds_s16x4_ptr)(tile + (kbase + 4) * stride + col));
    union {
      s16x4 h[2];
      bf16x8 v;
    } u;
    u.h[0] = lo;
    u.h[1] = hi;
    return u.v;
  };

  int const KT = (K + kBK - 1) / kBK;
  gload(0);
  lstore(0);
  __syncthreads();
  int cur = 0;
  for (int kt = 0; kt < KT; kt++) {
    bool const more = kt + 1 < KT;
    if (more) {
      gload((kt + 1) * kBK);
    }
#pragma unroll
    for (int kk = 0; kk < kBK / 16; kk++) {
      bf16x8 af[TM], bfr[TN];
#pragma unroll
      for (int i = 0; i < TM; i++) {
        af[i] = frag(As[cur], GA::kStride, TA, wm0 + i * 32, kk);
      }
#pragma unroll
      for (int j = 0; j < TN; j++) {
        bfr[j] = frag(Bs[cur], GB::kStride, TBL, wn0 + j * 32, kk);
      }
#pragma unroll
      for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bfr[j],
                                                             acc[i][j], 0, 0, 0);
    }
    if (more) {
      lstore(cur ^ 1);
    }
    __syncthreads();
    cur ^= 1;
  }

  // Epilogue: accumulator element r of lane l is row 8*(r/4) + 4*(l/32) + r%4,
  // column l % 32 of its 32x32 tile.
#pragma unroll
  for (int j = 0; j < TN; j++) {
    int const n = n0 + wn0 + j * 32 + (lane & 31);
    bool const n_ok = !EDGE || n < N;
    float bv = 0.0f;
    if (bias != nullptr && n_ok) {
      bv = VecIO<bf16>::load1(bias + n);
    }
#pragma unroll
    for (int i = 0; i < TM; i++) {
#pragma unroll
      for (int r = 0; r < 16; r++) {
        int const m = m0 + wm0 + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        if (n_ok && (!EDGE || m < M)) {
          float v = acc[i][j][r] + bv;
          v = apply_activation(v, act);
          bf16 *dst = C + (int64_t)m * ldc + n;
          if (accumulate) {
            v += VecIO<bf16>::load1(dst);
          }
          VecIO<bf16>::store1(dst, v);
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------
// bf16 MFMA kernel, pipelined variant for shapes that tile exactly:
//  * operand tiles go global -> LDS directly (global_load_lds_dwordx4, no VGPR
//    staging, no LDS write instructions) into a ring of STAGES buffers, so the
//    loads of the next STAGES-1 k-tiles are in flight while one is consumed --
//    this is what hides HBM/L2 latency when only one workgroup fits a CU;
//  * a direct load writes 64 lanes x 16 B contiguously, so bank conflicts are
//    avoided by permuting which 16-byte chunk each lane FETCHES (an XOR
//    swizzle) instead of padding rows;
//  * the accumulator tile is computed transposed (B as the first MFMA operand)
//    so that a lane holds 4 consecutive output columns, staged through LDS and
//    written to HBM as full 16-byte chunks with bias/activation/accumulate
//    applied on the way.
// ---------------------------------------------------------------------------
// PF = how many k-steps ahead of its use a fragment is read from LDS (PF + 1
// register buffers).  PF = 1 is what both tile configurations use; PF = 3 was
// measured on the 128x128 tile (2 MFMAs per k-step per wave) and gained nothing.
// Column sums add up blocks of 32 rows as four runs of 8 (colsum_partial_vec_kernel below).
constexpr int kColsumRowsPerLane = 8;
constexpr int kColsumRowsPerBlock = 4 * kColsumRowsPerLane;

struct GemmTailArgs {
  bf16 const *in;
  bf16 *out;
  DropoutParams dropout;
  // kTailDropoutGeluGrad only, optional: [M / 32][N] sums of 32-row blocks of
  // what the tail stores, added up in colsum_partial_vec_kernel's order
  float *colsum_partials;
};

// A second GEMM of the same kind and reduction length run by the same launch:
// workgroups from first_tiles on compute it.
struct GemmSecondProblem {
  bf16 const *A, *B;
  bf16 *C;
  int M, N;
  int64_t lda, ldb, ldc;
  int first_tiles;  // number of tiles (= workgroups) of the first problem
};

// TAIL (GemmEpilogue::Tail): element-wise operators applied to the 8-element
// pieces of the output tile on their way from LDS to memory.
// PAIR: the launch carries two problems (no bias, no split-K).
template <int BM, int BN, int WM, int WN, int BK, int STAGES, int PF, bool TA, bool TB, int TAIL = 0,
          bool PAIR = false>
__global__ __launch_bounds__((BM / WM) * (BN / WN) * 64) void gemm_bf16_pipe_kernel(
    bf16 const *__restrict__ A, bf16 const *__restrict__ B, bf16 *C, int M,
    int N, int K, int64_t lda, int64_t ldb, int64_t ldc,
    bf16 const *__restrict__ bias, int act, int accumulate,
    float *__restrict__ partial, int k_tiles_per_split, GemmTailArgs tail, GemmSecondProblem second) {
  int bid = blockIdx.x;
  if constexpr (PAIR) {
    if (bid >= second.first_tiles) {  // uniform over the workgroup
      bid -= second.first_tiles;
      A = second.A, B = second.B, C = second.C;
      M = second.M, N = second.N;
      lda = second.lda, ldb = second.ldb, ldc = second.ldc;
    }
  }
  // partial != nullptr: split-K.  Workgroup (tile, split) reduces k-tiles
  // [split * k_tiles_per_split, +k_tiles_per_split) and stores its fp32
  // accumulators to partial[split][M][N]; a second kernel sums the splits and
  // applies the epilogue.
  constexpr int NW = (BM / WM) * (BN / WN);
  constexpr int NT = NW * 64;
  constexpr int TM = WM / 32, TN = WN / 32;
  constexpr bool TBL = (TB == false);  // B tile lies as [BK][BN]
  constexpr int A_ELEMS = BM * BK, B_ELEMS = BN * BK;
  constexpr int A_LOADS = A_ELEMS / 8 / NT, B_LOADS = B_ELEMS / 8 / NT;
  constexpr int LPT = A_LOADS + B_LOADS;  // direct loads per thread per k-tile
  constexpr int STAGE_ELEMS = A_ELEMS + B_ELEMS;
  constexpr int CPRK = BK / 8;             // 16-byte chunks per K-contiguous row
  constexpr int RPW = 256 / (BK * 2);      // K-contiguous rows per 256-byte bank window
  constexpr int CS = WN + 8;               // row stride of a wave's staged output tile
  static_assert(A_ELEMS / 8 % NT == 0 && B_ELEMS / 8 % NT == 0, "tile/threads");
  static_assert(STAGES * LPT <= 63, "vmcnt range");

  extern __shared__ __attribute__((aligned(16))) bf16 smem[];

  int const t = threadIdx.x, lane = t & 63, wave = t >> 6;
  int const wm0 = (wave / (BN / WN)) * WM;
  int const wn0 = (wave % (BN / WN)) * WN;
  int tm, tn;
  int const tiles = (M / BM) * (N / BN);
  int const split = partial != nullptr ? bid / tiles : 0;
  tile_coords(partial != nullptr ? bid % tiles : bid, M / BM, N / BN, tm, tn);
  int const m0 = tm * BM, n0 = tn * BN;
  int const kt0 = split * k_tiles_per_split;  // first k-tile of this workgroup

  // Per-lane offset of its first chunk inside the block's operand panel; the
  // chunk of load i lies a uniform number of rows further on, and the k-tile
  // advances a uniform base, so a load address is a scalar base plus one
  // 32-bit lane offset that never changes.
  // K-contiguous tile [rows][BK]: physical chunk pc of a row holds logical
  // chunk pc ^ ((row / RPW) % CPRK).  Tile lying as [BK][cols]: the 64-byte
  // segment s of row k sits at segment s ^ (k % 4).
  constexpr int ROWS_PER_LOAD_KC = NT / CPRK;     // rows covered by one load of all threads
  static_assert((ROWS_PER_LOAD_KC / RPW) % CPRK == 0, "swizzle must repeat per load");
  static_assert((!TA || (NT * 8 % BM == 0 && (NT * 8 / BM) % 4 == 0)) && (!TBL || (NT * 8 % BN == 0 && (NT * 8 / BN) % 4 == 0)),
                "a panel lying [BK][cols] must divide into whole loads, and the swizzle repeat per load");
  unsigned voff_a, voff_b;
  {
    int c = wave * 64 + lane;
    if (!TA) {
      int row = c / CPRK, pc = c % CPRK;
      int lc = pc ^ ((row / RPW) & (CPRK - 1));
      voff_a = (unsigned)(row * lda + lc * 8) * 2u;
    } else {
      constexpr int CPR = BM / 8;
      int krow = c / CPR, pc = c % CPR;
      int lc = ((((pc >> 2) ^ (krow & 3)) << 2) | (pc & 3));
      voff_a = (unsigned)(krow * lda + lc * 8) * 2u;
    }
    if (!TBL) {
      int row = c / CPRK, pc = c % CPRK;
      int lc = pc ^ ((row / RPW) & (CPRK - 1));
      voff_b = (unsigned)(row * ldb + lc * 8) * 2u;
    } else {
      constexpr int CPR = BN / 8;
      int krow = c / CPR, pc = c % CPR;
      int lc = ((((pc >> 2) ^ (krow & 3)) << 2) | (pc & 3));
      voff_b = (unsigned)(krow * ldb + lc * 8) * 2u;
    }
  }
  int64_t const step_a = TA ? (int64_t)(NT * 8 / BM) * lda : (int64_t)ROWS_PER_LOAD_KC * lda;
  int64_t const step_b = TBL ? (int64_t)(NT * 8 / BN) * ldb : (int64_t)ROWS_PER_LOAD_KC * ldb;
  bf16 const *const panel_a = TA ? A + m0 : A + (int64_t)m0 * lda;
  bf16 const *const panel_b = TBL ? B + n0 : B + (int64_t)n0 * ldb;

  // LDS destinations of the direct loads are scalar byte addresses: base + stage + chunk row
  unsigned const smem_addr = lds_address_of(smem);
  int const wave_s = __builtin_amdgcn_readfirstlane(wave);
  // Loads [first, first + count) of a k-tile's LPT direct loads (A's, then B's).
  // (first and count are constants once the caller's loops are unrolled)
  auto issue_some = [&](int kt, int stage, int first, int count) __attribute__((always_inline)) {
    unsigned const sa = smem_addr + (unsigned)(stage * STAGE_ELEMS) * 2u;
    unsigned const sb = sa + (unsigned)A_ELEMS * 2u;
    i32x4 const ra = buffer_resource(panel_a + (TA ? (int64_t)(kt0 + kt) * BK * lda : (int64_t)(kt0 + kt) * BK));
    i32x4 const rb = buffer_resource(panel_b + (TBL ? (int64_t)(kt0 + kt) * BK * ldb : (int64_t)(kt0 + kt) * BK));
#pragma unroll
    for (int q = 0; q < LPT; q++) {
      if (q < first || q >= first + count) continue;
      if (q < A_LOADS) {
        lds_dma16(ra, voff_a, (unsigned)(q * step_a) * 2u, sa + (unsigned)(q * NW + wave_s) * 1024u);
      } else {
        int const i = q - A_LOADS;
        lds_dma16(rb, voff_b, (unsigned)(i * step_b) * 2u, sb + (unsigned)(i * NW + wave_s) * 1024u);
      }
    }
  };
  auto issue = [&](int kt, int stage) {
    issue_some(kt, stage, 0, LPT);
  };

  // Fragment readers (see the layouts above).  Everything lane-dependent in
  // an LDS address is tabulated once here; inside the loop an address is
  // stage base + table entry + a compile-time constant that folds into the
  // instruction's offset field, so the k-loop carries almost no address math.
  constexpr int KS = BK / 16;  // MFMA k-steps per tile
  // K-contiguous tile: lane l reads row (row0 + l%32), logical chunk 2 kk + l/32.
  // row0 is a multiple of 32, so the swizzle term depends on the lane only.
  int kc_off[KS];
  {
    int const sw = ((lane & 31) / RPW) & (CPRK - 1);
#pragma unroll
    for (int kk = 0; kk < KS; kk++) {
      kc_off[kk] = (lane & 31) * BK + (((2 * kk + (lane >> 5)) ^ sw) << 3);
    }
  }
  auto frag_kc = [&](bf16 const *tile, int row0, int kk) -> bf16x8 {
    return *reinterpret_cast<bf16x8 const *>(tile + kc_off[kk] + row0 * BK);
  };
  // Tile lying as [BK][cols]: lane reads rows kk*16 + 8 (l/32) + (l%16)/4 (+4),
  // columns col0 + 16 ((l/16)%2) + 4 (l%4); the 64-byte segment index is
  // XOR-ed with (row % 4), which touches only its two low bits.
  int tr_tab_a[4], tr_tab_b[4];
  {
    int const i16 = lane & 15;
    int const q = i16 >> 2;
    int const inseg = ((lane >> 4) & 1) * 16 + (i16 & 3) * 4;
    int const krow = (lane >> 5) * 8 + q;
#pragma unroll
    for (int c = 0; c < 4; c++) {
      tr_tab_a[c] = krow * BM + ((c ^ q) << 5) + inseg;
      tr_tab_b[c] = krow * BN + ((c ^ q) << 5) + inseg;
    }
  }
  auto frag_tr = [&](bf16 const *tile, int rowlen, int const (&tab)[4], int col0, int kk) -> bf16x8 {
    int const seg = col0 >> 5;
    bf16 const *p = tile + tab[seg & 3] + ((seg & ~3) << 5) + kk * 16 * rowlen;
    typedef s16x4 __attribute__((address_space(3))) * lds_s16x4_ptr;
    s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p));
    s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p + 4 * rowlen));
    union {
      s16x4 h[2];
      bf16x8 v;
    } u;
    u.h[0] = lo;
    u.h[1] = hi;
    return u.v;
  };

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

  int const KT = partial != nullptr ? k_tiles_per_split : K / BK;
  constexpr int NB = PF + 1;  // fragment buffers
  static_assert(KS % NB == 0, "buffer index must not depend on the tile");
  static_assert(STAGES >= 2, "one stage in use, at least one in flight");
  // With three or more stages a refill is not issued in one burst after the
  // barrier that frees its stage, but in KS equal parts: part 0 after that
  // barrier, part j in k-step j-1 of the following tile.  A burst of LPT loads
  // from every wave at once overruns the memory pipeline's instruction queue;
  // a wave that cannot issue its next load cannot issue its next MFMA either.
  constexpr bool SPREAD = STAGES >= 3 && LPT % KS == 0;
  constexpr int PART = SPREAD ? LPT / KS : LPT;
  // One wave per SIMD and two stages: a refill goes out in two halves, the first behind the
  // barrier that frees its stage, the second in the first k-step of the following tile.
  constexpr bool WIDE2 = WM == 128 && (WN == 128 || WN == 96) && STAGES == 2;
  constexpr int PRO_PART = WIDE2 ? LPT / 2 : PART;  // of the last tile the prologue starts
#pragma unroll
  for (int s = 0; s < STAGES; s++) {
    if (s < KT) {
      if ((SPREAD || WIDE2) && s == STAGES - 1) {
        issue_some(s, s, 0, PRO_PART);  // tile 0's steps issue the rest
      } else {
        issue(s, s);
      }
    }
  }
  // Fragments are double-buffered in registers: while the MFMAs of one k-step
  // run, the LDS reads of the next step (of the next tile, at a tile's last
  // step) are already in flight.
  bf16x8 af[NB][TM], bfr[NB][TN];
  auto read_frags = [&](int buf, int stage, int kk) {
    bf16 const *sa = smem + stage * STAGE_ELEMS;
    bf16 const *sb = sa + A_ELEMS;
#pragma unroll
    for (int i = 0; i < TM; i++) {
      af[buf][i] = TA ? frag_tr(sa, BM, tr_tab_a, wm0 + i * 32, kk) : frag_kc(sa, wm0 + i * 32, kk);
    }
#pragma unroll
    for (int j = 0; j < TN; j++) {
      bfr[buf][j] = TBL ? frag_tr(sb, BN, tr_tab_b, wn0 + j * 32, kk) : frag_kc(sb, wn0 + j * 32, kk);
    }
  };
  // Tile 0 must have landed (STAGES-1 younger tiles may still be in flight).
  if (STAGES - 1 < KT) {
    wait_vmcnt<(STAGES - 2) * LPT + PRO_PART>();
  } else {
    wait_vmcnt<0>();
  }
  // Barrier without a memory fence: a fence would wait for every direct load
  // still in flight; the vmcnt waits already cover the tile that is needed.
  asm volatile("s_barrier" ::: "memory");
#pragma unroll
  for (int kk = 0; kk < PF; kk++) read_frags(kk, 0, kk);
  // One k-tile.  STEADY: every condition of the generic body is known true
  // (next tile exists, a refill is due, STAGES-2 younger tiles in flight), so
  // the steady-state loop is branch-free.
  // SST: the tile's stage when the caller knows it (the steady loop, unrolled by STAGES), -1
  // otherwise.  With the stage a constant every LDS address of the tile is a loop-invariant
  // register plus an immediate; computed from kt it costs three vector instructions per k-step,
  // which two waves on a SIMD do not get for free.
  auto tile_step = [&](int kt, auto steady_tag, auto stage_tag) {
    constexpr bool STEADY = decltype(steady_tag)::value;
    constexpr int SST = decltype(stage_tag)::value;
    auto stage_at = [&](int d) { return SST >= 0 ? (SST + d) % STAGES : (kt + d) % STAGES; };
    int const stage = stage_at(0);
    if constexpr (WIDE2) {
      // One wave per SIMD: nothing but this wave's own instruction order hides a latency, so
      // the order is written out.  A k-step is 16 MFMAs.  Behind each of them sits one of the 8
      // fragment reads of the next step or one of up to 8 direct loads, alternating, fenced so
      // that the compiler keeps them there.  The refill of a stage goes out in two halves: the
      // first behind the barrier that frees the stage (last step of its tile), the second in
      // step 0 of the following tile; the steps in between carry fragment reads only.
      static_assert(PF == 1 && TM == 4 && (TN == 4 || TN == 3) && LPT % 2 == 0 && KS >= 2, "written for these shapes");
      // A k-step has NS = TM * TN MFMAs; behind them go the NR = TM + TN fragment reads of the
      // next step and, in the two steps that carry them, NL = LPT / 2 direct loads, each kind
      // spread evenly over the slots with the loads half a spacing behind the reads (4 x 4
      // blocks: reads in the even slots, loads in the odd ones; 4 x 3: twelve slots for seven
      // reads and seven loads).
      constexpr int NS = TM * TN, NR = TM + TN, NL = LPT / 2;
#pragma unroll
      for (int kk = 0; kk < KS; kk++) {
        int const cur = kk % NB, nxt = (kk + PF) % NB;
        bool const within = kk + PF < KS;            // the next step lies in this tile
        bool const reads = within || STEADY || kt + 1 < KT;
        int const rstage = within ? stage : stage_at(1);
        int const rkk = within ? kk + PF : kk + PF - KS;
        bf16 const *ra = smem + rstage * STAGE_ELEMS;
        bf16 const *rb = ra + A_ELEMS;
        bool const loads = kk == 0 ? (STEADY || kt + 1 < KT) : !within ? (STEADY || kt + 2 < KT) : false;
        int const ltile = kk == 0 ? kt + 1 : kt + 2;
        int const lstage = kk == 0 ? stage_at(1) : stage;
        int const lfirst = kk == 0 ? LPT / 2 : 0;
        // slot p follows MFMA p.  Even slots: a fragment read, in the order in which the next
        // step's MFMAs (row block by row block) first use the fragments: A0, B0..B3, A1, A2, A3.
        // Odd slots: a direct load.
        auto aux = [&](int p) __attribute__((always_inline)) {
          // (all reads first, then the loads, measured 2-7% slower: the four waves' reads then
          // meet in the LDS pipeline in bursts)
#pragma unroll
          for (int r = 0; r < NR; r++) {
            if (r * NS / NR != p || !reads) continue;
            if (r == 0 || r > TN) {
              int const i = r == 0 ? 0 : r - TN;
              af[nxt][i] = TA ? frag_tr(ra, BM, tr_tab_a, wm0 + i * 32, rkk) : frag_kc(ra, wm0 + i * 32, rkk);
            } else {
              int const j = r - 1;
              bfr[nxt][j] = TBL ? frag_tr(rb, BN, tr_tab_b, wn0 + j * 32, rkk) : frag_kc(rb, wn0 + j * 32, rkk);
            }
          }
#pragma unroll
          for (int l = 0; l < NL; l++) {
            if ((2 * l + 1) * NS / (2 * NL) != p || !loads) continue;
            issue_some(ltile, lstage, lfirst + l, 1);
          }
        };
        __builtin_amdgcn_sched_barrier(0);
        acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[cur][0], af[cur][0], acc[0][0], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        if (!within && reads) {
          // the next tile must have landed (nothing younger is in flight with two stages) and
          // every wave must be done reading this one
          wait_vmcnt<0>();
          asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        }
#pragma unroll
        for (int m = 1; m < TM * TN; m++) {
          aux(m - 1);
          __builtin_amdgcn_sched_barrier(0);
          acc[m / TN][m % TN] =
              __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[cur][m % TN], af[cur][m / TN], acc[m / TN][m % TN], 0, 0, 0);
          __builtin_amdgcn_sched_barrier(0);
        }
        aux(TM * TN - 1);
      }
      return;
    }
#pragma unroll
    for (int kk = 0; kk < KS; kk++) {
      int const cur = kk % NB;
      int const nxt = (kk + PF) % NB;  // buffer of the step read now
      // The first MFMA of the step is issued before the prefetch below so that
      // the wait for this step's fragments does not also cover the reads
      // issued now (the hardware counter is in order).
      __builtin_amdgcn_sched_barrier(0);
      acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[cur][0], af[cur][0], acc[0][0], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
      if (SPREAD && kk + 1 < KS) {
        // part kk+1 of the tile that goes into the stage freed one tile ago
        if (STEADY || kt + STAGES - 1 < KT) {
          issue_some(kt + STAGES - 1, stage_at(STAGES - 1), (kk + 1) * PART, PART);
        }
      }
      if (kk + PF < KS) {
        read_frags(nxt, stage, kk + PF);
      } else if (STEADY || kt + 1 < KT) {
        if (kk + PF == KS) {
          // First read of tile kt+1: make it visible and refill this tile's own
          // stage -- under this step's MFMAs, which cover those latencies.
          // Every wave has all fragments of tile kt in registers once its LDS
          // counter drains, so after the barrier the stage is free.
          if (STEADY || kt + STAGES - 1 < KT) {
            wait_vmcnt<(STAGES - 2) * LPT>();
          } else {
            wait_vmcnt<0>();
          }
          asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
          if (STEADY || kt + STAGES < KT) {
            issue_some(kt + STAGES, stage, 0, PART);
          }
        }
        read_frags(nxt, stage_at(1), kk + PF - KS);
      }
      __builtin_amdgcn_sched_barrier(0);
      // Transposed accumulation: rows of the MFMA result = output columns.
#pragma unroll
      for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
          if (i + j > 0)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[cur][j], af[cur][i], acc[i][j], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  using Dyn = std::integral_constant<int, -1>;
  int kt = 0;
  if constexpr (!WIDE2 && (STAGES == 4 || STAGES == 2)) {
    for (; kt + 2 * STAGES - 1 < KT; kt += STAGES) {  // kt % STAGES == 0, all STAGES tiles steady
      tile_step(kt, std::true_type{}, std::integral_constant<int, 0>{});
      tile_step(kt + 1, std::true_type{}, std::integral_constant<int, 1>{});
      if constexpr (STAGES == 4) {
        tile_step(kt + 2, std::true_type{}, std::integral_constant<int, 2>{});
        tile_step(kt + 3, std::true_type{}, std::integral_constant<int, 3>{});
      }
    }
  }
  for (; kt + STAGES < KT; kt++) {
    tile_step(kt, std::true_type{}, Dyn{});
  }
  for (; kt < KT; kt++) {
    tile_step(kt, std::false_type{}, Dyn{});
  }
  // acc[i][j][r]: output row m = wm0 + 32 i + lane % 32,
  //               column n = wn0 + 32 j + 8 (r / 4) + 4 (lane / 32) + r % 4.
  // The plain store (no tail, nothing to add to): straight from the registers.  A lane holds
  // columns 8 g + 4 h .. + 3 of every group g of 8 (h = its lane half); one swap of the lane
  // halves per pair of groups gives the lower half the 8 columns of group g and the upper half
  // those of group g + 1, so that every lane stores 16 bytes and the two halves together 32
  // contiguous bytes of a row.  No LDS, so no barrier either: a wave writes its tile as soon as
  // its own loop is done.  Used by the one-wave-per-SIMD kernel, where it is 4-6% of a launch at
  // reductions up to 2048 (FFN-up shape 37.6 -> 36.0 us); with two waves per SIMD the staged
  // epilogue below, whose stores are whole 128-byte lines, is 2-5% ahead.  (The 32-byte pieces
  // cost memory traffic: 49 MB written per 32 MB tile set by the write counter, whatever the
  // order of the stores; going row by row instead of column block by column block is 3% slower.)
  if constexpr (TAIL == GemmEpilogue::kTailNone && WIDE2) {
    if (partial == nullptr && accumulate == 0) {  // uniform over the launch
      auto direct = [&](auto actf) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < TN; j++) {
          float bv[4][4];
#pragma unroll
          for (int g = 0; g < 4; g++) {
            u32x2 raw = {0u, 0u};
            if (bias != nullptr) raw = *reinterpret_cast<u32x2 const *>(bias + n0 + wn0 + j * 32 + 8 * g + 4 * (lane >> 5));
            bv[g][0] = __uint_as_float(raw[0] << 16);
            bv[g][1] = __uint_as_float(raw[0] & 0xffff0000u);
            bv[g][2] = __uint_as_float(raw[1] << 16);
            bv[g][3] = __uint_as_float(raw[1] & 0xffff0000u);
          }
#pragma unroll
          for (int i = 0; i < TM; i++) {
            bf16 *const row = C + (int64_t)(m0 + wm0 + i * 32 + (lane & 31)) * ldc + n0 + wn0 + j * 32 + 8 * (lane >> 5);
#pragma unroll
            for (int g = 0; g < 4; g += 2) {
              uint32_t w[2][2];
#pragma unroll
              for (int gg = 0; gg < 2; gg++) {
                float v[4];
#pragma unroll
                for (int e = 0; e < 4; e++) v[e] = actf(acc[i][j][4 * (g + gg) + e] + bv[g + gg][e]);
                w[gg][0] = pack_bf16x2(v[0], v[1]);
                w[gg][1] = pack_bf16x2(v[2], v[3]);
              }
              // swaps the upper lane half of the first operand with the lower half of the second
              auto const lo = __builtin_amdgcn_permlane32_swap(w[0][0], w[1][0], false, false);
              auto const hi = __builtin_amdgcn_permlane32_swap(w[0][1], w[1][1], false, false);
              u32x4 const out = {lo[0], hi[0], lo[1], hi[1]};
              *reinterpret_cast<u32x4 *>(row + 8 * g) = out;
            }
          }
        }
      };
      direct([](float v) { return v; });  // (this kernel is only launched without an activation)
      return;
    }
  }
  __syncthreads();  // all stages are free now: reuse them for the output tile

  // Each wave stages its own WM x WN tile and writes it out in 16-byte chunks.
  bf16 *cs = smem + wave * (WM * CS);
  constexpr int CCH = WM * WN / 8 / 64;  // 16-byte chunks per lane
  // The activation is a compile-time functor here: a per-element switch inside
  // the unrolled loops made the epilogue several times longer than the GEMM's
  // own store traffic.
  auto finish = [&](auto actf) __attribute__((always_inline)) {
    bf16 *const dst = C;
    bool const add_old = accumulate != 0;
    // A wave stages and writes out its own tile, so only its own LDS accesses have to be ordered,
    // and those complete in program order: no barrier.  With one wave per SIMD (128x128 wave tiles)
    // the tile goes out in two halves of 64 rows, so that the stores of the first half are under
    // way while the second is converted.
    constexpr int HALVES = WIDE2 ? 2 : 1;
    constexpr int TMH = TM / HALVES;
#pragma unroll
    for (int half = 0; half < HALVES; half++) {
    // The lane's bias values depend on (j, g, lane / 32) only: they are
    // fetched once per (j, g) and used for the row blocks.
#pragma unroll
    for (int j = 0; j < TN; j++) {
#pragma unroll
      for (int g = 0; g < 4; g++) {
        int const n = j * 32 + 8 * g + 4 * (lane >> 5);
        u32x2 raw = {0u, 0u};
        if (bias != nullptr) raw = *reinterpret_cast<u32x2 const *>(bias + n0 + wn0 + n);
        float const bv[4] = {__uint_as_float(raw[0] << 16), __uint_as_float(raw[0] & 0xffff0000u),
                             __uint_as_float(raw[1] << 16), __uint_as_float(raw[1] & 0xffff0000u)};
#pragma unroll
        for (int i = half * TMH; i < (half + 1) * TMH; i++) {
          int const m = i * 32 + (lane & 31);
          float v[4];
#pragma unroll
          for (int e = 0; e < 4; e++) v[e] = acc[i][j][4 * g + e] + bv[e];
#pragma unroll
          for (int e = 0; e < 4; e++) v[e] = actf(v[e]);
          if (add_old) {
            // add the old value in fp32 before the single rounding
            u32x2 old = *reinterpret_cast<u32x2 const *>(dst + (int64_t)(m0 + wm0 + m) * ldc + n0 + wn0 + n);
            v[0] += __uint_as_float(old[0] << 16);
            v[1] += __uint_as_float(old[0] & 0xffff0000u);
            v[2] += __uint_as_float(old[1] << 16);
            v[3] += __uint_as_float(old[1] & 0xffff0000u);
          }
          u32x2 w = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
          *reinterpret_cast<u32x2 *>(cs + m * CS + n) = w;
        }
      }
    }
#pragma unroll
    for (int i = half * (CCH / HALVES); i < (half + 1) * (CCH / HALVES); i++) {
      int c = lane + i * 64;
      int row = c / (WN / 8), ch = c % (WN / 8);
      u32x4 v = *reinterpret_cast<u32x4 const *>(cs + row * CS + ch * 8);
      int64_t const at = (int64_t)(m0 + wm0 + row) * ldc + n0 + wn0 + ch * 8;
      if constexpr (TAIL == GemmEpilogue::kTailNone) {
        *reinterpret_cast<u32x4 *>(dst + at) = v;
      } else {
        // ldc == N here: `at` is the element's index in the dense tensor, and
        // the piece is one block of the dropout stream
        uint32_t w[4];
        philox4x32_10((tail.dropout.offset + (uint64_t)at) >> 3, tail.dropout.key, w);
        u32x4 aux = {0u, 0u, 0u, 0u};
        if constexpr (TAIL == GemmEpilogue::kTailGeluDropout) {
          *reinterpret_cast<u32x4 *>(dst + at) = v;
        } else {
          aux = *reinterpret_cast<u32x4 const *>(tail.in + at);
        }
        u32x4 r;
#pragma unroll
        for (int q = 0; q < 4; q++) {
          float x[2] = {__uint_as_float(v[q] << 16), __uint_as_float(v[q] & 0xffff0000u)};
          float const a[2] = {__uint_as_float(aux[q] << 16), __uint_as_float(aux[q] & 0xffff0000u)};
#pragma unroll
          for (int h = 0; h < 2; h++) {
            if constexpr (TAIL == GemmEpilogue::kTailGeluDropout) {
              x[h] = storage_round<bf16>(gelu_forward(x[h]));
            }
            x[h] = keep(w, 2 * q + h, tail.dropout) ? x[h] * tail.dropout.scale : 0.0f;
            if constexpr (TAIL == GemmEpilogue::kTailDropoutGeluGrad) {
              x[h] = storage_round<bf16>(x[h]) * gelu_derivative(a[h]);
            }
            if constexpr (TAIL == GemmEpilogue::kTailDropoutAdd) {
              x[h] = storage_round<bf16>(x[h]) + a[h];
            }
          }
          r[q] = pack_bf16x2(x[0], x[1]);
        }
        bf16 *const to = TAIL == GemmEpilogue::kTailGeluDropout ? tail.out : dst;
        *reinterpret_cast<u32x4 *>(to + at) = r;
        if constexpr (TAIL == GemmEpilogue::kTailDropoutGeluGrad) {
          // kept for the column sums below (the lane's own piece: no other lane reads it before the barrier)
          if (tail.colsum_partials != nullptr) *reinterpret_cast<u32x4 *>(cs + row * CS + ch * 8) = r;
        }
      }
    }
    }  // half
    if constexpr (TAIL == GemmEpilogue::kTailDropoutGeluGrad) {
      if (tail.colsum_partials != nullptr) {  // uniform over the launch
        __syncthreads();
        // A lane owns a column of the wave's tile; per block of 32 rows: four
        // runs of 8 rows summed in row order, then (0 + 1) + (2 + 3).
        for (int col = lane; col < WN; col += 64) {
#pragma unroll
          for (int blk = 0; blk < WM / kColsumRowsPerBlock; blk++) {
            float run[4];
#pragma unroll
            for (int q = 0; q < 4; q++) {
              float acc_rows = 0.0f;
#pragma unroll
              for (int r = 0; r < kColsumRowsPerLane; r++) {
                acc_rows += VecIO<bf16>::load1(cs + (blk * kColsumRowsPerBlock + q * kColsumRowsPerLane + r) * CS + col);
              }
              run[q] = acc_rows;
            }
            int64_t const part = (m0 + wm0) / kColsumRowsPerBlock + blk;
            tail.colsum_partials[part * N + n0 + wn0 + col] = (run[0] + run[1]) + (run[2] + run[3]);
          }
        }
      }
    }
  };
  // One wave per SIMD with a 128x128 wave tile keeps 256 accumulator registers: only the plain
  // epilogue (bias, no activation, no split-K) is compiled for it, so that nothing outside the
  // loop competes for registers.
  if constexpr (WIDE2) {
    finish([](float v) { return v; });
    return;
  }
  if (partial != nullptr) {
    // raw accumulators, 16 bytes (4 consecutive columns) per store
    float *dst = partial + (int64_t)split * M * N;
#pragma unroll
    for (int i = 0; i < TM; i++) {
      int64_t const m = m0 + wm0 + i * 32 + (lane & 31);
#pragma unroll
      for (int j = 0; j < TN; j++) {
#pragma unroll
        for (int g = 0; g < 4; g++) {
          int const n = n0 + wn0 + j * 32 + 8 * g + 4 * (lane >> 5);
          f32x4 v = {acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
          *reinterpret_cast<f32x4 *>(dst + m * N + n) = v;
        }
      }
    }
    return;
  }
  if (act == FFK_ACT_NONE) {
    finish([](float v) { return v; });
  } else if (act == FFK_ACT_GELU) {
    finish([](float v) { return gelu_forward(v); });
  } else if (act == FFK_ACT_RELU) {
    finish([](float v) { return v >= 0.0f ? v : 0.0f; });
  } else {
    finish([act](float v) { return apply_activation(v, act); });
  }
}

// Second pass of split-K: C = epilogue(sum over splits of partial[s][M][N]).
__global__ __launch_bounds__(256) void splitk_reduce_kernel(
    float const *__restrict__ partial, int splits, int M, int N, bf16 *C,
    int64_t ldc, bf16 const *__restrict__ bias, int act, int accumulate) {
  int64_t const q = (int64_t)blockIdx.x * 256 + threadIdx.x;
  int64_t const total = (int64_t)M * N;
  if (q * 4 >= total) return;
  int64_t const m = (q * 4) / N;
  int const n = (int)((q * 4) % N);
  f32x4 s = *reinterpret_cast<f32x4 const *>(partial + q * 4);
  for (int k = 1; k < splits; k++) {
    f32x4 v = *reinterpret_cast<f32x4 const *>(partial + k * total + q * 4);
    s += v;
  }
  bf16 *dst = C + m * ldc + n;
  float v[4] = {s[0], s[1], s[2], s[3]};
#pragma unroll
  for (int e = 0; e < 4; e++) {
    if (bias != nullptr) v[e] += VecIO<bf16>::load1(bias + n + e);
    v[e] = apply_activation(v[e], act);
  }
  if (accumulate) {
    u32x2 old = *reinterpret_cast<u32x2 const *>(dst);
    v[0] += __uint_as_float(old[0] << 16);
    v[1] += __uint_as_float(old[0] & 0xffff0000u);
    v[2] += __uint_as_float(old[1] << 16);
    v[3] += __uint_as_float(old[1] & 0xffff0000u);
  }
  u32x2 w = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
  *reinterpret_cast<u32x2 *>(dst) = w;
}

template <int BM, int BN, int WM, int WN, int BK, int STAGES>
struct PipeCfg {
  static constexpr int NW = (BM / WM) * (BN / WN);
  static constexpr size_t kStageBytes = (size_t)STAGES * (BM + BN) * BK * sizeof(bf16);
  static constexpr size_t kOutBytes = (size_t)NW * WM * (WN + 8) * sizeof(bf16);
  static constexpr size_t kLds = kStageBytes > kOutBytes ? kStageBytes : kOutBytes;
  static_assert(kLds <= 160 * 1024, "LDS budget");
};

template <int BM, int BN, int WM, int WN, int BK, int STAGES, int PF, bool TA, bool TB, int TAIL = 0>
static hipError_t launch_pipe(hipStream_t st, bf16 const *A, bf16 const *B,
                              bf16 *C, int M, int N, int K, int64_t lda,
                              int64_t ldb, int64_t ldc, GemmEpilogue const &ep,
                              int splits = 1) {
  using Cfg = PipeCfg<BM, BN, WM, WN, BK, STAGES>;
  constexpr int NT = Cfg::NW * 64;
  if (describe_only("gemm_bf16_pipe_kernel<%d,%d,%d,%d,%d,%d,%d,%s,%s,%d,false>%s", BM, BN, WM, WN, BK, STAGES, PF,
                    tf(TA), tf(TB), TAIL, splits > 1 ? " (split-K) + splitk_reduce_kernel" : "")) {
    return hipSuccess;
  }
  auto kern = gemm_bf16_pipe_kernel<BM, BN, WM, WN, BK, STAGES, PF, TA, TB, TAIL>;
  GemmTailArgs const tail = {static_cast<bf16 const *>(ep.tail_in), static_cast<bf16 *>(ep.tail_out),
                             ep.tail_dropout, ep.tail_colsum_partials};
  static LdsOptIn lds;  // per template instance
  if (hipError_t e = lds.ensure(reinterpret_cast<void const *>(kern), (int)Cfg::kLds); e != hipSuccess) return e;
  int const blocks = (M / BM) * (N / BN);
  if (splits > 1) {
    float *partial = static_cast<float *>(ep.splitk_ws);
    kern<<<blocks * splits, NT, Cfg::kLds, st>>>(A, B, C, M, N, K, lda, ldb, ldc, nullptr,
                                                FFK_ACT_NONE, 0, partial, K / BK / splits, tail,
                                                GemmSecondProblem{});
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    int64_t const quads = (int64_t)M * N / 4;
    splitk_reduce_kernel<<<(unsigned)ceil_div(quads, 256), 256, 0, st>>>(
        partial, splits, M, N, C, ldc, static_cast<bf16 const *>(ep.bias), ep.activation,
        ep.accumulate);
    return hipGetLastError();
  }
  kern<<<blocks, NT, Cfg::kLds, st>>>(A, B, C, M, N, K, lda, ldb, ldc,
                                     static_cast<bf16 const *>(ep.bias), ep.activation,
                                     ep.accumulate, nullptr, 0, tail, GemmSecondProblem{});
  return hipGetLastError();
}

// Two GEMMs of the same kind and reduction length on 128x128 tiles in one launch.
template <bool TA, bool TB>
static hipError_t launch_pipe_pair(hipStream_t st, GemmProblem const &p0, GemmProblem const &p1, int K,
                                   bool accumulate) {
  using Cfg = PipeCfg<128, 128, 64, 32, 64, 4>;
  constexpr int NT = Cfg::NW * 64;
  auto kern = gemm_bf16_pipe_kernel<128, 128, 64, 32, 64, 4, 1, TA, TB, 0, true>;
  static LdsOptIn lds;
  if (hipError_t e = lds.ensure(reinterpret_cast<void const *>(kern), (int)Cfg::kLds); e != hipSuccess) return e;
  int const t0 = (int)((p0.M / 128) * (p0.N / 128)), t1 = (int)((p1.M / 128) * (p1.N / 128));
  GemmSecondProblem const second = {static_cast<bf16 const *>(p1.A), static_cast<bf16 const *>(p1.B),
                                    static_cast<bf16 *>(p1.C), (int)p1.M, (int)p1.N, p1.lda, p1.ldb, p1.ldc, t0};
  kern<<<t0 + t1, NT, Cfg::kLds, st>>>(static_cast<bf16 const *>(p0.A), static_cast<bf16 const *>(p0.B),
                                       static_cast<bf16 *>(p0.C), (int)p0.M, (int)p0.N, K, p0.lda, p0.ldb, p0.ldc,
                                       nullptr, FFK_ACT_NONE, accumulate ? 1 : 0, nullptr, 0, GemmTailArgs{}, second);
  return hipGetLastError();
}

// ---------------------------------------------------------------------------
// fp32 MFMA kernel (32x32x2), 64x64 block tile, bounds-checked everywhere.
// ---------------------------------------------------------------------------
template <bool TA, bool TB>
__global__ __launch_bounds__(256) void gemm_f32_kernel(
    float const *__restrict__ A, float const *__restrict__ B, float *C, int M,
    int N, int K, int64_t lda, int64_t ldb, int64_t ldc,
    float const *__restrict__ bias, int act, int accumulate) {
  constexpr int BM = 64, BN = 64, BKF = 16, LD = 68;
  __shared__ float As[BKF][LD];  // [k][m]
  __shared__ float Bs[BKF][LD];  // [k][n]
  int const t = threadIdx.x;
  int const lane = t & 63;
  int const wave = t >> 6;
  int const wm0 = (wave >> 1) * 32;
  int const wn0 = (wave & 1) * 32;
  int const nbn = (N + BN - 1) / BN;
  int const m0 = (blockIdx.x / nbn) * BM;
  int const n0 = (blockIdx.x % nbn) * BN;

  f32x16 acc;
#pragma unroll
  for (int r = 0; r < 16; r++) acc[r] = 0.0f;

  for (int k0 = 0; k0 < K; k0 += BKF) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      int m, k;
      if (!TA) {  // A[M,K]: k fastest across lanes
        k = t & 15;
        m = (t >> 4) + 16 * i;
      } else {  // A[K,M]: m fastest
        m = t & 63;
        k = (t >> 6) + 4 * i;
      }
      int gm = m0 + m, gk = k0 + k;
      float v = 0.0f;
      if (gm < M && gk < K) {
        v = TA ? A[(int64_t)gk * lda + gm] : A[(int64_t)gm * lda + gk];
      }
      As[k][m] = v;
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
      int n, k;
      if (TB) {  // B[N,K]: k fastest
        k = t & 15;
        n = (t >> 4) + 16 * i;
      } else {  // B[K,N]: n fastest
        n = t & 63;
        k = (t >> 6) + 4 * i;
      }
      int gn = n0 + n, gk = k0 + k;
      float v = 0.0f;
      if (gn < N && gk < K) {
        v = TB ? B[(int64_t)gn * ldb + gk] : B[(int64_t)gk * ldb + gn];
      }
      Bs[k][n] = v;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < BKF / 2; kk++) {
      float a = As[2 * kk + (lane >> 5)][wm0 + (lane & 31)];
      float b = Bs[2 * kk + (lane >> 5)][wn0 + (lane & 31)];
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc, 0, 0, 0);
    }
    __syncthreads();
  }

  int const n = n0 + wn0 + (lane & 31);
  if (n < N) {
    float bv = bias != nullptr ? bias[n] : 0.0f;
#pragma unroll
    for (int r = 0; r < 16; r++) {
      int const m = m0 + wm0 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
      if (m < M) {
        float v = apply_activation(acc[r] + bv, act);
        float *dst = C + (int64_t)m * ldc + n;
        if (accumulate) {
          v += *dst;
        }
        *dst = v;
      }
    }
  }
}

// ---------------------------------------------------------------------------
// fp32 MFMA kernel for operands that can be read 16 bytes at a time: 128 x BN
// block tile (BN = 128 or 64), 2 x 2 waves of 64 x BN/2, reduction tiles of 32.
// The next tile travels global -> registers while this one is multiplied and
// goes to the other LDS buffer afterwards: one barrier per tile.  The fp32
// MFMA (32x32x2, 64 cycles) is so slow next to its two one-register operands
// that LDS and issue bandwidth are never short; what the kernel has to do is
// keep loads in flight and the matrix pipe fed, which two workgroups per CU and
// fragments read one step ahead take care of.
//   An operand whose reduction index is contiguous in memory (A[M,K], B[N,K])
// lies in LDS as [k / 2][row][k % 2], row stride 2 * rows + 4: a lane's four
// consecutive k go out as two 8-byte writes, and the MFMA read -- lanes 0-31
// one k, lanes 32-63 the next -- touches 64 consecutive floats.  The compiler
// pairs a lane's reads for two 32-row blocks into one two-dword read, which is
// served 32 lanes at a time: the pairs of odd blocks are stored swapped, so
// that those 32 lanes take even banks for one block and odd banks for the
// other (unswapped they met in the same banks: 2.6 conflict cycles per cycle
// of LDS work, the matrix pipe 80% busy).  An operand
// whose rows are contiguous (A[K,M], B[K,N]) lies as [k][row] with the two
// 32-float halves of every odd k swapped, which does the same for the read
// without padding.  Every element's products are added in ascending k, two per
// MFMA, as in gemm_f32_kernel: the two kernels give the same bits.
// Rows and columns past the edge are read from the last valid ones and never
// stored; k past the end is zeroed when the tile is written to LDS.
// ---------------------------------------------------------------------------
template <bool TA, bool TB, int BN>
__global__ __launch_bounds__(256, 2) void gemm_f32_tiled_kernel(
    float const *__restrict__ A, float const *__restrict__ B, float *C, int M, int N, int K, int64_t lda,
    int64_t ldb, int64_t ldc, float const *__restrict__ bias, int act, int accumulate) {
  constexpr int BM = 128, BKT = 32;
  constexpr int TNW = BN / 64;              // 32-column blocks per wave
  constexpr bool A_KC = !TA, B_KC = TB;     // reduction index contiguous in memory
  constexpr int A_CH = BM * BKT / 4 / 256, B_CH = BN * BKT / 4 / 256;  // 16-byte chunks per thread and tile
  constexpr int A_SP = 2 * BM + 4, B_SP = 2 * BN + 4;                  // pair-layout row strides
  constexpr int A_FLOATS = A_KC ? (BKT / 2) * A_SP : BKT * BM;
  constexpr int B_FLOATS = B_KC ? (BKT / 2) * B_SP : BKT * BN;
  __shared__ __attribute__((aligned(16))) float As[2][A_FLOATS];
  __shared__ __attribute__((aligned(16))) float Bs[2][B_FLOATS];
  int const t = threadIdx.x, lane = t & 63, wave = t >> 6;
  int const h = lane >> 5, l32 = lane & 31;
  int const wm0 = (wave >> 1) * 64, wn0 = (wave & 1) * (BN / 2);
  int tm, tn;
  tile_coords(blockIdx.x, (M + BM - 1) / BM, (N + BN - 1) / BN, tm, tn);
  int const m0 = tm * BM, n0 = tn * BN;

  // Chunk i of this thread: (row, k quad) of a k-contiguous operand, (k row, row quad) otherwise.
  // Its address for k-tile 0 is kept and moved on by a constant per tile; only a tile that
  // reaches past K (the last one of a ragged reduction) computes clamped addresses afresh.
  constexpr int NCH = A_CH + B_CH;
  f32x4 rgs[2][NCH];  // k-tile kt travels in set kt % 2, two tiles ahead of its use
  float const *pg[NCH];
#pragma unroll
  for (int i = 0; i < A_CH; i++) {
    int const c = t + i * 256;
    pg[i] = A_KC ? A + (int64_t)min(m0 + c / 8, M - 1) * lda + 4 * (c % 8)
                 : A + (int64_t)(c / (BM / 4)) * lda + min(m0 + 4 * (c % (BM / 4)), M - 4);
  }
#pragma unroll
  for (int i = 0; i < B_CH; i++) {
    int const c = t + i * 256;
    pg[A_CH + i] = B_KC ? B + (int64_t)min(n0 + c / 8, N - 1) * ldb + 4 * (c % 8)
                        : B + (int64_t)(c / (BN / 4)) * ldb + min(n0 + 4 * (c % (BN / 4)), N - 4);
  }
  int64_t const step_a = A_KC ? BKT : (int64_t)BKT * lda, step_b = B_KC ? BKT : (int64_t)BKT * ldb;
  // load of chunk i of k-tile kt; pg[i] points at k-tile kt on entry and at kt + 1 on return
  auto gload_chunk = [&](int kt, int i, f32x4 (&rg)[NCH]) __attribute__((always_inline)) {
    int const k0 = kt * BKT;
    bool const is_a = i < A_CH;
    if (k0 + BKT <= K) {
      rg[i] = *reinterpret_cast<f32x4 const *>(pg[i]);
    } else {
      int const c = t + (is_a ? i : i - A_CH) * 256;
      // how far this chunk's k lies past the last one it may read
      if (is_a ? A_KC : B_KC) {
        int const over = max(k0 + 4 * (c % 8) - (K - 4), 0);
        rg[i] = *reinterpret_cast<f32x4 const *>(pg[i] - over);
      } else {
        int const over = max(k0 + c / ((is_a ? BM : BN) / 4) - (K - 1), 0);
        rg[i] = *reinterpret_cast<f32x4 const *>(pg[i] - (int64_t)over * (is_a ? lda : ldb));
      }
    }
    pg[i] += is_a ? step_a : step_b;
  };
  auto gload = [&](int kt, f32x4 (&rg)[NCH]) {
#pragma unroll
    for (int i = 0; i < NCH; i++) gload_chunk(kt, i, rg);
  };
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  // chunk i of k-tile kt from its registers into buffer buf, k past the end zeroed
  auto lstore_chunk = [&](int buf, int kt, int i, f32x4 const (&rg)[NCH]) __attribute__((always_inline)) {
    f32x4 const zero = {0.0f, 0.0f, 0.0f, 0.0f};
    int const k0 = kt * BKT;
    bool const is_a = i < A_CH;
    int const c = t + (is_a ? i : i - A_CH) * 256;
    float *dst = is_a ? As[buf] : Bs[buf];
    int const SP = is_a ? A_SP : B_SP, R = is_a ? BM : BN;
    // (vector instructions between the MFMAs are not free: with two waves on a SIMD the masks
    // and selects of this function, applied to every tile, cost 5-10% of the matrix pipe's time.
    // The mask is for the one tile that reaches past K; which blocks are swapped is known per chunk.)
    bool const whole = k0 + BKT <= K;  // uniform
    if (is_a ? A_KC : B_KC) {
      int const row = c / 8, kq = c % 8;
      f32x4 v = rg[i];
      if (!whole) {
        asm volatile("" ::: "memory");  // a branch, not four selects on every tile
        v = k0 + 4 * kq < K ? v : zero;
      }
      // odd 32-row blocks hold their k pairs swapped; row / 32 = chunk number (t / 8 < 32)
      bool const odd = (((is_a ? i : i - A_CH) & 1) != 0);
      *reinterpret_cast<f32x2 *>(&dst[(2 * kq) * SP + 2 * row]) = odd ? f32x2{v[1], v[0]} : f32x2{v[0], v[1]};
      *reinterpret_cast<f32x2 *>(&dst[(2 * kq + 1) * SP + 2 * row]) = odd ? f32x2{v[3], v[2]} : f32x2{v[2], v[3]};
    } else {
      int const k = c / (R / 4), rq = c % (R / 4);
      f32x4 v = rg[i];
      if (!whole) {
        asm volatile("" ::: "memory");
        v = k0 + k < K ? v : zero;
      }
      *reinterpret_cast<f32x4 *>(&dst[k * R + ((4 * rq) ^ ((k & 1) * 32))]) = v;
    }
  };
  // operand value of this lane for MFMA step kk (k = 2 kk + h) and its row
  auto frag_a = [&](int buf, int kk, int row) -> float {
    return A_KC ? As[buf][kk * A_SP + 2 * row + (h ^ ((row >> 5) & 1))] : As[buf][(2 * kk + h) * BM + (row ^ (h * 32))];
  };
  auto frag_b = [&](int buf, int kk, int row) -> float {
    return B_KC ? Bs[buf][kk * B_SP + 2 * row + (h ^ ((row >> 5) & 1))] : Bs[buf][(2 * kk + h) * BN + (row ^ (h * 32))];
  };

  f32x16 acc[2][TNW];
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < TNW; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

  int const KT = (K + BKT - 1) / BKT;
  gload(0, rgs[0]);
  if (KT > 1) gload(1, rgs[1]);
#pragma unroll
  for (int i = 0; i < NCH; i++) lstore_chunk(0, 0, i, rgs[0]);
  __syncthreads();
  // One k-tile, kt, from buffer kt % 2.  AHEAD2: k-tile kt + 2 exists; its loads go out one per
  // step in the first NCH steps (a burst of them holds the wave, and with it its MFMAs, for as
  // long as the memory pipeline takes to accept them), into the register set that tile kt
  // travelled in.  AHEAD1: k-tile kt + 1
  // exists; it was asked for a tile ago and is written to the other buffer (which nobody reads
  // during this tile) one chunk per step in the last NCH steps, under the MFMAs.  A wave sits
  // at each MFMA until the pipe takes it, so whatever is placed between two of them costs
  // nothing as long as it is short; the fences keep it there.
  constexpr int KS = BKT / 2;
  static_assert(NCH <= KS, "one chunk per step");
  auto tile = [&](int kt, auto set_tag, auto ahead1_tag, auto ahead2_tag) {
    constexpr int SET = decltype(set_tag)::value;  // = kt % 2
    constexpr bool AHEAD1 = decltype(ahead1_tag)::value, AHEAD2 = decltype(ahead2_tag)::value;
    float af[2][2], bfv[2][TNW];
#pragma unroll
    for (int i = 0; i < 2; i++) af[0][i] = frag_a(SET, 0, wm0 + i * 32 + l32);
#pragma unroll
    for (int j = 0; j < TNW; j++) bfv[0][j] = frag_b(SET, 0, wn0 + j * 32 + l32);
#pragma unroll
    for (int kk = 0; kk < KS; kk++) {
      int const c = kk & 1, nx = c ^ 1;
      // the next step's fragments are asked for before this step's MFMAs are issued: reads
      // issued behind them would start their round trip only when the last one has gone
      if (kk + 1 < KS) {
#pragma unroll
        for (int i = 0; i < 2; i++) af[nx][i] = frag_a(SET, kk + 1, wm0 + i * 32 + l32);
#pragma unroll
        for (int j = 0; j < TNW; j++) bfv[nx][j] = frag_b(SET, kk + 1, wn0 + j * 32 + l32);
      }
      __builtin_amdgcn_sched_barrier(0);
      acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[c][0], bfv[c][0], acc[0][0], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
      if (AHEAD2 && kk < NCH) gload_chunk(kt + 2, kk, rgs[SET]);
      if (AHEAD1 && kk >= KS - NCH) lstore_chunk(SET ^ 1, kt + 1, kk - (KS - NCH), rgs[SET ^ 1]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < TNW; j++)
          if (i + j > 0) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[c][i], bfv[c][j], acc[i][j], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
    __syncthreads();
  };
  using T0 = std::integral_constant<int, 0>;
  using T1 = std::integral_constant<int, 1>;
  int kt = 0;
  for (; kt + 3 < KT; kt += 2) {  // both tiles of the pair have two successors
    tile(kt, T0{}, std::true_type{}, std::true_type{});
    tile(kt + 1, T1{}, std::true_type{}, std::true_type{});
  }
  // the last one to three tiles (kt is even)
  if (kt + 2 < KT) {
    tile(kt, T0{}, std::true_type{}, std::true_type{});
    tile(kt + 1, T1{}, std::true_type{}, std::false_type{});
    tile(kt + 2, T0{}, std::false_type{}, std::false_type{});
  } else if (kt + 1 < KT) {
    tile(kt, T0{}, std::true_type{}, std::false_type{});
    tile(kt + 1, T1{}, std::false_type{}, std::false_type{});
  } else {
    tile(kt, T0{}, std::false_type{}, std::false_type{});
  }

  // accumulator element r of lane l: row 8 (r / 4) + 4 (l / 32) + r % 4, column l % 32 of its block
#pragma unroll
  for (int j = 0; j < TNW; j++) {
    int const n = n0 + wn0 + j * 32 + l32;
    if (n >= N) continue;
    float const bv = bias != nullptr ? bias[n] : 0.0f;
#pragma unroll
    for (int i = 0; i < 2; i++) {
      int const mb = m0 + wm0 + i * 32 + 4 * h;
      float old[16];
      if (accumulate) {  // what C holds, all loads in flight together
#pragma unroll
        for (int r = 0; r < 16; r++) {
          int const m = min(mb + 8 * (r >> 2) + (r & 3), M - 1);
          old[r] = C[(int64_t)m * ldc + n];
        }
      }
#pragma unroll
      for (int r = 0; r < 16; r++) {
        int const m = mb + 8 * (r >> 2) + (r & 3);
        float v = apply_activation(acc[i][j][r] + bv, act);
        if (accumulate) v += old[r];
        if (m < M) C[(int64_t)m * ldc + n] = v;
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Plain kernel for bf16 shapes the tiled kernel cannot take.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void gemm_bf16_plain_kernel(
    bf16 const *__restrict__ A, bf16 const *__restrict__ B, bf16 *C, int M,
    int N, int K, int64_t lda, int64_t ldb, int64_t ldc, int ta, int tb,
    bf16 const *__restrict__ bias, int act, int accumulate) {
  int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (int64_t)M * N) return;
  int m = (int)(idx / N), n = (int)(idx % N);
  float acc = 0.0f;
  for (int k = 0; k < K; k++) {
    float a = VecIO<bf16>::load1(ta ? A + (int64_t)k * lda + m : A + (int64_t)m * lda + k);
    float b = VecIO<bf16>::load1(tb ? B + (int64_t)n * ldb + k : B + (int64_t)k * ldb + n);
    acc += a * b;
  }
  if (bias != nullptr) acc += VecIO<bf16>::load1(bias + n);
  acc = apply_activation(acc, act);
  bf16 *dst = C + (int64_t)m * ldc + n;
  if (accumulate) acc += VecIO<bf16>::load1(dst);
  VecIO<bf16>::store1(dst, acc);
}

template <int BM, int BN, int WM, int WN, bool TA, bool TB>
static hipError_t launch_bf16(hipStream_t st, bf16 const *A, bf16 const *B,
                              bf16 *C, int M, int N, int K, int64_t lda,
                              int64_t ldb, int64_t ldc, GemmEpilogue const &ep) {
  int const blocks = (int)(ceil_div(M, BM) * ceil_div(N, BN));
  constexpr int NT = (BM / WM) * (BN / WN) * 64;
  bool const edge = (M % BM) || (N % BN) || (K % kBK);
  bf16 const *bias = static_cast<bf16 const *>(ep.bias);
  if (describe_only("gemm_bf16_kernel<%d,%d,%d,%d,%s,%s,%s>", BM, BN, WM, WN, tf(TA), tf(TB), tf(edge))) return hipSuccess;
  if (edge) {
    gemm_bf16_kernel<BM, BN, WM, WN, TA, TB, true><<<blocks, NT, 0, st>>>(
        A, B, C, M, N, K, lda, ldb, ldc, bias, ep.activation, ep.accumulate);
  } else {
    gemm_bf16_kernel<BM, BN, WM, WN, TA, TB, false><<<blocks, NT, 0, st>>>(
        A, B, C, M, N, K, lda, ldb, ldc, bias, ep.activation, ep.accumulate);
  }
  return hipGetLastError();
}

// FFK_OPTION_GEMM_VARIANT = 128|256|1 forces a tile configuration (1 = the
// register-staged kernel); 0 = the heuristic.  For tuning runs and tests.
static int gemm_variant_override() { return option(FFK_OPTION_GEMM_VARIANT); }

// Number of K splits for an M x N output of 128x128 tiles: enough to give
// every CU a workgroup, each split at least 8 k-tiles of 64 long, and no more
// than the caller's scratch (splits * M * N floats) allows.
static int splitk_splits(int64_t M, int64_t N, int64_t K, size_t ws_bytes) {
  int64_t const tiles = (M / 128) * (N / 128);
  if (tiles <= 0 || tiles >= kNumCU / 2 || K % 64 != 0) return 1;
  int s = 1;
  while (s * 2 * tiles <= kNumCU && s < 8 && (K / 64) % (s * 2) == 0 && K / (s * 2) >= 512 &&
         (size_t)(s * 2) * (size_t)(M * N) * sizeof(float) <= ws_bytes) {
    s *= 2;
  }
  return s;
}

size_t gemm_splitk_workspace_bytes(int dtype, int64_t M, int64_t N, int64_t K) {
  if (dtype != FFK_BF16 || M % 128 != 0 || N % 128 != 0) return 0;
  int const s = splitk_splits(M, N, K, ~(size_t)0);
  return s > 1 ? (size_t)s * (size_t)(M * N) * sizeof(float) : 0;
}

// What every pipelined kernel asks of the operands, whatever its tile.
static bool pipe_operands_ok(bf16 const *C, int K, int64_t lda, int64_t ldb, int64_t ldc, GemmEpilogue const &ep) {
  bool const c_vec = (ldc % 8 == 0) && aligned16(C);
  // the pipelined kernels fetch the bias in 8-byte pieces
  bool const aux_ok = reinterpret_cast<uintptr_t>(ep.bias) % 8 == 0;
  // the direct loads address an operand panel with 32-bit byte offsets
  bool const panel_ok = 2 * 256 * std::max(lda, ldb) < (int64_t(1) << 31);
  return c_vec && aux_ok && panel_ok && K % 64 == 0;
}

// Which pipelined tile a bf16 GEMM runs on: 256, 128, or 0 (none of the two:
// split-K or the register-staged kernels).
static int pipe_tile_for(bf16 const *C, int M, int N, int K, int64_t lda, int64_t ldb, int64_t ldc,
                         GemmEpilogue const &ep, int variant) {
  if (!pipe_operands_ok(C, K, lda, ldb, ldc, ep) || variant == 1) return 0;
  bool const fits256 = M % 256 == 0 && N % 256 == 0;
  bool const fits128 = M % 128 == 0 && N % 128 == 0;
  int64_t const t256 = fits256 ? (int64_t)(M / 256) * (N / 256) : 0;
  int64_t const t128 = fits128 ? (int64_t)(M / 128) * (N / 128) : 0;
  // 256x256 tiles (8 waves of 128x64, four 32-deep stages of 32 KB whose
  // refills are spread over the k-steps) halve the L2->LDS traffic per flop;
  // they win whenever they still occupy most CUs.  Otherwise 128x128x64 tiles
  // with 8 waves of 64x32 keep two waves per SIMD on every CU.
  if ((variant == 0 && t256 >= kNumCU * 3 / 4) || ((variant == 256 || variant == 264) && fits256)) return 256;
  if ((variant == 0 && t128 >= kNumCU / 2) || (variant == 128 && fits128)) return 128;
  return 0;
}

template <bool TA, bool TB>
static hipError_t pick_bf16(hipStream_t st, bf16 const *A, bf16 const *B,
                            bf16 *C, int M, int N, int K, int64_t lda,
                            int64_t ldb, int64_t ldc, GemmEpilogue const &ep) {
  int const variant = gemm_variant_override();
  int const pipe_tile = pipe_tile_for(C, M, N, K, lda, ldb, ldc, ep, variant);
  {
    bool const fits128 = M % 128 == 0 && N % 128 == 0;
    bool const use256 = pipe_tile == 256, use128 = pipe_tile == 128;
    if (ep.tail != GemmEpilogue::kTailNone) {
      // gemm_tail_supported() has been asked: one of the two tiles fits
      if constexpr (!TA && TB) {
        constexpr int kTail = GemmEpilogue::kTailGeluDropout;
        if (ep.tail == kTail && use256) {
          return launch_pipe<256, 256, 128, 64, 32, 4, 1, TA, TB, kTail>(st, A, B, C, M, N, K, lda, ldb, ldc, ep);
        }
        if (ep.tail == kTail && use128) {
          return launch_pipe<128, 128, 64, 32, 64, 4, 1, TA, TB, kTail>(st, A, B, C, M, N, K, lda, ldb, ldc, ep);
        }
        constexpr int kAdd = GemmEpilogue::kTailDropoutAdd;
        if (ep.tail == kAdd && use256) {
          return launch_pipe<256, 256, 128, 64, 32, 4, 1, TA, TB, kAdd>(st, A, B, C, M, N, K, lda, ldb, ldc, ep);
        }
        if (ep.tail == kAdd && use128) {
          return launch_pipe<128, 128, 64, 32, 64, 4, 1, TA, TB, kAdd>(st, A, B, C, M, N, K, lda, ldb, ldc, ep);
        }
      }
      if constexpr (!TA && !TB) {
        constexpr int kTail = GemmEpilogue::kTailDropoutGeluGrad;
        if (ep.tail == kTail && use256) {
          return launch_pipe<256, 256, 128, 64, 32, 4, 1, TA, TB, kTail>(st, A, B, C, M, N, K, lda, ldb, ldc, ep);
        }
        if (ep.tail == kTail && use128) {
          return launch_pipe<128, 128, 64, 32, 64, 4, 1, TA, TB, kTail>(st, A, B, C, M, N, K, lda, ldb, ldc, ep);
        }
      }
      return hipErrorInvalidValue;
    }
    // An output that 256x256 tiles cover in a ragged last round but 256x192 tiles cover in whole
    // rounds of the chip (the attention block's fused Q/K/V projection: [4096, 3072] is 192 tiles of
    // the first kind on 256 CUs, 256 of the second): one wave per SIMD on 128x96 wave tiles.  Only
    // with both operands K-contiguous: a [K][192] panel does not divide into whole direct loads.
    if constexpr (!TA && TB) {
      bool const fits192 = M % 256 == 0 && N % 192 == 0;
      int64_t const t256 = M % 256 == 0 && N % 256 == 0 ? (int64_t)(M / 256) * (N / 256) : 0;
      int64_t const t192 = fits192 ? (int64_t)(M / 256) * (N / 192) : 0;
      bool const whole_rounds = t192 > 0 && t192 % kNumCU == 0 && t256 % kNumCU != 0;
      if (pipe_operands_ok(C, K, lda, ldb, ldc, ep) && variant != 1 && ep.activation == FFK_ACT_NONE && K >= 1024 &&
          (variant == 192 ? fits192 : (variant == 0 && whole_rounds))) {
        return launch_pipe<256, 192, 128, 96, 64, 2, 1, TA, TB>(st, A, B, C, M, N, K, lda, ldb, ldc, ep);
      }
    }
    // Reductions from 1024 on without an activation: one wave per SIMD on 128x128 wave tiles, two
    // 64-deep stages, every instruction of the loop placed by hand.  (Below that the eight-wave
    // kernel's shorter prologue weighs more than the faster loop.)
    if (use256 && ep.activation == FFK_ACT_NONE && (variant == 264 || (variant == 0 && K >= 1024))) {
      return launch_pipe<256, 256, 128, 128, 64, 2, 1, TA, TB>(st, A, B, C, M, N, K, lda, ldb, ldc, ep);
    }
    if (use256) {
      return launch_pipe<256, 256, 128, 64, 32, 4, 1, TA, TB>(st, A, B, C, M, N, K, lda, ldb, ldc, ep);
    }
    if (use128) {
      return launch_pipe<128, 128, 64, 32, 64, 4, 1, TA, TB>(st, A, B, C, M, N, K, lda, ldb, ldc, ep);
    }
    // Few output tiles and a long reduction: split K so every CU has a tile.
    bool const pipe_ok = pipe_tile_for(C, M, N, K, lda, ldb, ldc, ep, 128) == 128;  // but for the tile count
    int const splits = fits128 && pipe_ok ? splitk_splits(M, N, K, ep.splitk_ws_bytes) : 1;
    if (variant == 0 && splits > 1 && ep.splitk_ws != nullptr && aligned16(ep.splitk_ws)) {
      return launch_pipe<128, 128, 64, 32, 64, 4, 1, TA, TB>(st, A, B, C, M, N, K, lda, ldb, ldc, ep, splits);
    }
    // No scratch to split the reduction with: from 32 tiles and a reduction of 2048 on, the
    // pipelined tile on the CUs it reaches is still ahead of the register-staged 64x64 kernel on
    // four times as many ([1024,1024] over 4096 rows, 64 tiles: 30.5 against 34.5 us).
    if (variant == 0 && pipe_ok && fits128 && (int64_t)(M / 128) * (N / 128) >= kNumCU / 8 && K >= 2048) {
      return launch_pipe<128, 128, 64, 32, 64, 4, 1, TA, TB>(st, A, B, C, M, N, K, lda, ldb, ldc, ep);
    }
  }
  if (ep.tail != GemmEpilogue::kTailNone) return hipErrorInvalidValue;
  // Largest tile that still gives every CU a workgroup.
  int64_t const b128 = ceil_div(M, 128) * ceil_div(N, 128);
  if (b128 >= kNumCU) {
    return launch_bf16<128, 128, 64, 64, TA, TB>(st, A, B, C, M, N, K, lda, ldb, ldc, ep);
  }
  return launch_bf16<64, 64, 32, 32, TA, TB>(st, A, B, C, M, N, K, lda, ldb, ldc, ep);
}

// ---------------------------------------------------------------------------
// Column sums (bias gradient): out[n] (+)= sum_m X[m,n]
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void colsum_partial_kernel(
    T const *__restrict__ X, int64_t ldx, int M, int N, int rows_per_split,
    float *__restrict__ partials) {
  __shared__ float red[4][64];
  int const cx = threadIdx.x & 63;
  int const ry = threadIdx.x >> 6;
  int const n = blockIdx.x * 64 + cx;
  int const r0 = blockIdx.y * rows_per_split;
  int const r1 = min(M, r0 + rows_per_split);
  float s = 0.0f;
  if (n < N) {
    for (int m = r0 + ry; m < r1; m += 4) {
      s += VecIO<T>::load1(X + (int64_t)m * ldx + n);
    }
  }
  red[ry][cx] = s;
  __syncthreads();
  if (ry == 0 && n < N) {
    partials[(int64_t)blockIdx.y * N + n] =
        red[0][cx] + red[1][cx] + red[2][cx] + red[3][cx];
  }
}

// Vectorised first pass: a thread reads 16 bytes (8 bf16 / 4 fp32 columns) of
// kColsumRowsPerLane rows, all loads independent; 64 threads span the columns,
// the 4 row lanes of the workgroup meet in LDS.

// DROP: X is the gradient of a dropout's output; what is summed is the
// dropout's backward of it, rounded as stored, which is also written to G
// (dense, ldx == N: a lane's V elements are a Philox block or half of one).
template <typename T, bool DROP>
__global__ __launch_bounds__(256) void colsum_partial_vec_kernel(
    T const *__restrict__ X, int64_t ldx, int M, int N, int rows_per_split,
    float *__restrict__ partials, T *__restrict__ G, DropoutParams drop) {
  constexpr int V = VecIO<T>::kVec;
  __shared__ float red[4][64][V + 1];
  int const cx = threadIdx.x & 63;
  int const ry = threadIdx.x >> 6;
  int const n = (blockIdx.x * 64 + cx) * V;
  int const r0 = blockIdx.y * rows_per_split;
  int const r1 = min(M, r0 + rows_per_split);
  float s[V];
#pragma unroll
  for (int e = 0; e < V; e++) s[e] = 0.0f;
  if (n < N) {
    for (int m0 = r0 + ry * kColsumRowsPerLane; m0 < r1; m0 += kColsumRowsPerBlock) {
      float v[kColsumRowsPerLane][V];
#pragma unroll
      for (int i = 0; i < kColsumRowsPerLane; i++) {
        int const m = min(m0 + i, r1 - 1);  // clamped rows are masked below
        VecIO<T>::load_stream(X + (int64_t)m * ldx + n, v[i]);
      }
#pragma unroll
      for (int i = 0; i < kColsumRowsPerLane; i++) {
        if (m0 + i < r1) {
          if constexpr (DROP) {
            uint64_t const e0 = drop.offset + (uint64_t)(m0 + i) * (uint64_t)N + (uint64_t)n;
            uint32_t w[4];
            philox4x32_10(e0 >> 3, drop.key, w);
            if (V == 4 && (e0 & 4)) {  // upper half of the block
              w[0] = w[2];
              w[1] = w[3];
            }
#pragma unroll
            for (int e = 0; e < V; e++) v[i][e] = storage_round<T>(keep(w, e, drop) ? v[i][e] * drop.scale : 0.0f);
            VecIO<T>::store(G + (int64_t)(m0 + i) * ldx + n, v[i]);
          }
#pragma unroll
          for (int e = 0; e < V; e++) s[e] += v[i][e];
        }
      }
    }
  }
#pragma unroll
  for (int e = 0; e < V; e++) red[ry][cx][e] = s[e];
  __syncthreads();
  if (ry == 0 && n < N) {
#pragma unroll
    for (int e = 0; e < V; e++) {
      partials[(int64_t)blockIdx.y * N + n + e] =
          (red[0][cx][e] + red[1][cx][e]) + (red[2][cx][e] + red[3][cx][e]);
    }
  }
}

static int colsum_splits(int64_t M) {
  int64_t s = ceil_div(M, kColsumRowsPerBlock);
  return (int)(s < 1 ? 1 : (s > 256 ? 256 : s));
}

// Rows that one partial sum of the vector column-sum kernel covers.
static int64_t colsum_rows_per_split(int64_t M) {
  int64_t const rows = ceil_div(M, (int64_t)colsum_splits(M));
  return ceil_div(rows, (int64_t)kColsumRowsPerBlock) * kColsumRowsPerBlock;
}

int colsum_finish(hipStream_t st, int dtype, float const *partials, int64_t M, int64_t N, void *out,
                  bool accumulate) {
  FFK_REQUIRE(dtype == FFK_BF16 && M % kColsumRowsPerBlock == 0 && colsum_rows_per_split(M) == kColsumRowsPerBlock,
              "colsum_finish: partials of this shape do not come from a GEMM tail");
  FFK_HIP(colreduce_launch<bf16>(st, partials, (int)(M / kColsumRowsPerBlock), (int)N, (int)N,
                                 static_cast<bf16 *>(out), nullptr, accumulate));
  return FFK_OK;
}

int64_t colsum_partials_elems(int64_t M, int64_t N) {
  return (int64_t)colsum_splits(M) * N;
}

// dropped != nullptr: the sums are taken over dropout_backward(X), which is
// written to dropped; vector shapes only (FFK_ERR_UNSUPPORTED otherwise, before
// any launch).
template <typename T>
static int colsum_typed(hipStream_t st, T const *X, int64_t ldx, int64_t M,
                        int64_t N, T *out, bool accumulate, float *partials,
                        T *dropped = nullptr, DropoutParams const *drop = nullptr) {
  constexpr int V = VecIO<T>::kVec;
  int const splits = colsum_splits(M);
  int rows_per_split = (int)ceil_div(M, splits);
  bool const vec = (N % V == 0) && (ldx % V == 0) && aligned16(X);
  if (dropped != nullptr) {
    if (!vec || ldx != N || !aligned16(dropped) || (drop->offset & 7) != 0 || M >= (1ll << 31) || N >= (1ll << 31)) {
      return FFK_ERR_UNSUPPORTED;
    }
    rows_per_split = (int)(ceil_div(rows_per_split, kColsumRowsPerBlock) * kColsumRowsPerBlock);
    int const used = (int)ceil_div(M, rows_per_split);
    dim3 grid((unsigned)ceil_div(N, 64 * V), (unsigned)used);
    colsum_partial_vec_kernel<T, true><<<grid, 256, 0, st>>>(X, ldx, (int)M, (int)N, rows_per_split, partials,
                                                            dropped, *drop);
    FFK_CHECK_LAUNCH();
    FFK_HIP(colreduce_launch<T>(st, partials, used, (int)N, (int)N, out, nullptr, accumulate));
    return FFK_OK;
  }
  if (vec) {
    // whole row blocks per split so that only the last split has a ragged end
    rows_per_split = (int)(ceil_div(rows_per_split, kColsumRowsPerBlock) * kColsumRowsPerBlock);
    int const used = (int)ceil_div(M, rows_per_split);
    dim3 grid((unsigned)ceil_div(N, 64 * V), (unsigned)used);
    colsum_partial_vec_kernel<T, false><<<grid, 256, 0, st>>>(X, ldx, (int)M, (int)N, rows_per_split, partials,
                                                             nullptr, DropoutParams{});
    FFK_CHECK_LAUNCH();
    FFK_HIP(colreduce_launch<T>(st, partials, used, (int)N, (int)N, out, nullptr, accumulate));
    return FFK_OK;
  }
  dim3 grid((unsigned)ceil_div(N, 64), (unsigned)splits);
  colsum_partial_kernel<T><<<grid, 256, 0, st>>>(X, ldx, (int)M, (int)N, rows_per_split, partials);
  FFK_CHECK_LAUNCH();
  FFK_HIP(colreduce_launch<T>(st, partials, splits, (int)N, (int)N, out, nullptr, accumulate));
  return FFK_OK;
}

int colsum_dispatch(hipStream_t st, int dtype, void const *X, int64_t ldx,
                    int64_t M, int64_t N, void *out, bool accumulate,
                    float *partials) {
  FFK_REQUIRE(partials != nullptr, "colsum: partials scratch is NULL");
  if (dtype == FFK_FLOAT) {
    return colsum_typed<float>(st, static_cast<float const *>(X), ldx, M, N,
                               static_cast<float *>(out), accumulate, partials);
  }
  if (dtype == FFK_BF16) {
    return colsum_typed<bf16>(st, static_cast<bf16 const *>(X), ldx, M, N,
                              static_cast<bf16 *>(out), accumulate, partials);
  }
  return fail(FFK_ERR_UNSUPPORTED, "colsum: dtype %d not supported", dtype);
}

int dropout_backward_colsum(hipStream_t st, int dtype, void const *dy, void *dx, int64_t M, int64_t N,
                            void *colsum, bool accumulate, float *partials, DropoutParams const &drop) {
  FFK_REQUIRE(dy && dx && colsum && partials, "dropout_backward_colsum: NULL operand");
  FFK_REQUIRE(M > 0 && N > 0, "dropout_backward_colsum: non-positive dimension");
  if (dtype == FFK_FLOAT) {
    return colsum_typed<float>(st, static_cast<float const *>(dy), N, M, N, static_cast<float *>(colsum),
                               accumulate, partials, static_cast<float *>(dx), &drop);
  }
  if (dtype == FFK_BF16) {
    return colsum_typed<bf16>(st, static_cast<bf16 const *>(dy), N, M, N, static_cast<bf16 *>(colsum),
                              accumulate, partials, static_cast<bf16 *>(dx), &drop);
  }
  return FFK_ERR_UNSUPPORTED;
}

static bool pair_member_ok(bool ta, bool tb, GemmProblem const &p, int64_t K) {
  if (p.M <= 0 || p.N <= 0 || p.M % 128 != 0 || p.N % 128 != 0 || !p.A || !p.B || !p.C) return false;
  if (p.M >= (1ll << 31) || p.N >= (1ll << 31)) return false;
  if (p.lda < (ta ? p.M : K) || p.ldb < (tb ? K : p.N) || p.ldc < p.N) return false;
  bool const vec_ok = (p.lda % 8 == 0) && (p.ldb % 8 == 0) && aligned16(p.A) && aligned16(p.B);
  GemmEpilogue none;
  return vec_ok && pipe_tile_for(static_cast<bf16 const *>(p.C), (int)p.M, (int)p.N, (int)K, p.lda, p.ldb, p.ldc, none,
                                 128) == 128;
}

bool gemm_pair_supported(int dtype, bool ta, bool tb, int64_t K, GemmProblem const &p0, GemmProblem const &p1) {
  if (dtype != FFK_BF16 || K <= 0 || K % 64 != 0 || K >= (1ll << 31) || gemm_variant_override() != 0) return false;
  if (!pair_member_ok(ta, tb, p0, K) || !pair_member_ok(ta, tb, p1, K)) return false;
  // worth it when neither problem fills the chip on its own and the two together come closer
  int64_t const t0 = (p0.M / 128) * (p0.N / 128), t1 = (p1.M / 128) * (p1.N / 128);
  return t0 < 2 * kNumCU && t1 < 2 * kNumCU && t0 + t1 >= kNumCU / 2;
}

int gemm_dispatch_pair(hipStream_t st, int dtype, bool ta, bool tb, int64_t K, GemmProblem const &p0,
                       GemmProblem const &p1, bool accumulate) {
  FFK_REQUIRE(gemm_pair_supported(dtype, ta, tb, K, p0, p1),
              "gemm: these two problems do not run as one launch (ask gemm_pair_supported first)");
  hipError_t e;
  if (!ta && !tb) e = launch_pipe_pair<false, false>(st, p0, p1, (int)K, accumulate);
  else if (!ta && tb) e = launch_pipe_pair<false, true>(st, p0, p1, (int)K, accumulate);
  else if (ta && !tb) e = launch_pipe_pair<true, false>(st, p0, p1, (int)K, accumulate);
  else e = launch_pipe_pair<true, true>(st, p0, p1, (int)K, accumulate);
  FFK_HIP(e);
  return FFK_OK;
}

bool gemm_tail_supported(int dtype, bool ta, bool tb, int64_t M, int64_t N, int64_t K,
                         void const *A, int64_t lda, void const *B, int64_t ldb,
                         void const *C, int64_t ldc, GemmEpilogue const &ep) {
  if (dtype != FFK_BF16 || ta || ep.accumulate || ldc != N || M <= 0 || N <= 0 || K <= 0) return false;
  if (M >= (1ll << 31) || N >= (1ll << 31) || K >= (1ll << 31)) return false;
  if ((ep.tail_dropout.offset & 7) != 0) return false;
  if (ep.tail == GemmEpilogue::kTailGeluDropout) {
    if (!tb || ep.tail_out == nullptr || !aligned16(ep.tail_out)) return false;
  } else if (ep.tail == GemmEpilogue::kTailDropoutGeluGrad) {
    if (tb || ep.tail_in == nullptr || !aligned16(ep.tail_in)) return false;
    if (ep.tail_colsum_partials != nullptr && colsum_rows_per_split(M) != kColsumRowsPerBlock) return false;
  } else if (ep.tail == GemmEpilogue::kTailDropoutAdd) {
    if (!tb || ep.tail_in == nullptr || !aligned16(ep.tail_in)) return false;
  } else {
    return false;
  }
  bool const vec_ok = (K % 8 == 0) && (lda % 8 == 0) && (ldb % 8 == 0) && aligned16(A) && aligned16(B) &&
                      (tb || N % 8 == 0);
  return vec_ok && pipe_tile_for(static_cast<bf16 const *>(C), (int)M, (int)N, (int)K, lda, ldb, ldc, ep,
                                 gemm_variant_override()) != 0;
}

int gemm_dispatch(hipStream_t st, int dtype, bool ta, bool tb, int64_t M,
                  int64_t N, int64_t K, void const *A, int64_t lda,
                  void const *B, int64_t ldb, void *C, int64_t ldc,
                  GemmEpilogue const &ep) {
  FFK_REQUIRE(M >= 0 && N >= 0 && K >= 0, "gemm: negative dimension");
  if (M == 0 || N == 0) return FFK_OK;
  FFK_REQUIRE(A && B && C, "gemm: NULL operand");
  FFK_REQUIRE(M < (1ll << 31) && N < (1ll << 31) && K < (1ll << 31),
              "gemm: dimension exceeds 2^31");
  FFK_REQUIRE(lda >= (ta ? M : K) && ldb >= (tb ? K : N) && ldc >= N,
              "gemm: leading dimension smaller than the row length");
  hipError_t e;
  if (dtype == FFK_FLOAT) {
    FFK_REQUIRE(ep.tail == GemmEpilogue::kTailNone, "gemm: fused tails exist for bf16 only");
    float const *a = static_cast<float const *>(A);
    float const *b = static_cast<float const *>(B);
    float *c = static_cast<float *>(C);
    float const *bias = static_cast<float const *>(ep.bias);
    // 16-byte reads: aligned rows, and whole quads along whichever index is contiguous
    bool const tiled = aligned16(A) && aligned16(B) && lda % 4 == 0 && ldb % 4 == 0 && K >= 4 &&
                       (ta ? M % 4 == 0 && M >= 4 : K % 4 == 0) && (tb ? K % 4 == 0 : N % 4 == 0 && N >= 4) &&
                       M * N >= 128 * 128;
    if (tiled) {
      // 128 x 128 tiles when they give every CU two workgroups, 128 x 64 otherwise
      bool const wide = ceil_div(M, 128) * ceil_div(N, 128) >= 2 * kNumCU;
      int const tblocks = (int)(ceil_div(M, 128) * ceil_div(N, wide ? 128 : 64));
      if (describe_only("gemm_f32_tiled_kernel<%s,%s,%d>", tf(ta), tf(tb), wide ? 128 : 64)) return FFK_OK;
#define FFK_LAUNCH_F32T(TA_, TB_)                                              \
  do {                                                                         \
    if (wide)                                                                  \
      gemm_f32_tiled_kernel<TA_, TB_, 128><<<tblocks, 256, 0, st>>>(           \
          a, b, c, (int)M, (int)N, (int)K, lda, ldb, ldc, bias, ep.activation, ep.accumulate); \
    else                                                                       \
      gemm_f32_tiled_kernel<TA_, TB_, 64><<<tblocks, 256, 0, st>>>(            \
          a, b, c, (int)M, (int)N, (int)K, lda, ldb, ldc, bias, ep.activation, ep.accumulate); \
  } while (0)
      if (!ta && !tb) FFK_LAUNCH_F32T(false, false);
      else if (!ta && tb) FFK_LAUNCH_F32T(false, true);
      else if (ta && !tb) FFK_LAUNCH_F32T(true, false);
      else FFK_LAUNCH_F32T(true, true);
#undef FFK_LAUNCH_F32T
      FFK_CHECK_LAUNCH();
      return FFK_OK;
    }
    int const blocks = (int)(ceil_div(M, 64) * ceil_div(N, 64));
#define FFK_LAUNCH_F32(TA_, TB_)                                               \
  gemm_f32_kernel<TA_, TB_><<<blocks, 256, 0, st>>>(                           \
      a, b, c, (int)M, (int)N, (int)K, lda, ldb, ldc, bias, ep.activation,     \
      ep.accumulate)
    if (describe_only("gemm_f32_kernel<%s,%s>", tf(ta), tf(tb))) return FFK_OK;
    if (!ta && !tb) FFK_LAUNCH_F32(false, false);
    else if (!ta && tb) FFK_LAUNCH_F32(false, true);
    else if (ta && !tb) FFK_LAUNCH_F32(true, false);
    else FFK_LAUNCH_F32(true, true);
#undef FFK_LAUNCH_F32
    e = hipGetLastError();
  } else if (dtype == FFK_BF16) {
    FFK_REQUIRE(ep.tail == GemmEpilogue::kTailNone ||
                    gemm_tail_supported(dtype, ta, tb, M, N, K, A, lda, B, ldb, C, ldc, ep),
                "gemm: this shape has no fused tail (ask gemm_tail_supported first)");
    bf16 const *a = static_cast<bf16 const *>(A);
    bf16 const *b = static_cast<bf16 const *>(B);
    bf16 *c = static_cast<bf16 *>(C);
    // 16-byte chunks: K and any contiguous non-reduction extent must be a
    // multiple of 8 elements, rows 16-byte aligned.
    bool vec_ok = (K % 8 == 0) && (lda % 8 == 0) && (ldb % 8 == 0) &&
                  aligned16(A) && aligned16(B) && (!ta || M % 8 == 0) &&
                  (tb || N % 8 == 0) && K > 0;
    if (!vec_ok) {
      int64_t total = M * N;
      if (describe_only("gemm_bf16_plain_kernel")) return FFK_OK;
      gemm_bf16_plain_kernel<<<(unsigned)ceil_div(total, 256), 256, 0, st>>>(
          a, b, c, (int)M, (int)N, (int)K, lda, ldb, ldc, ta, tb,
          static_cast<bf16 const *>(ep.bias), ep.activation, ep.accumulate);
      e = hipGetLastError();
    } else if (!ta && !tb) {
      e = pick_bf16<false, false>(st, a, b, c, (int)M, (int)N, (int)K, lda, ldb, ldc, ep);
    } else if (!ta && tb) {
      e = pick_bf16<false, true>(st, a, b, c, (int)M, (int)N, (int)K, lda, ldb, ldc, ep);
    } else if (ta && !tb) {
      e = pick_bf16<true, false>(st, a, b, c, (int)M, (int)N, (int)K, lda, ldb, ldc, ep);
    } else {
      e = pick_bf16<true, true>(st, a, b, c, (int)M, (int)N, (int)K, lda, ldb, ldc, ep);
    }
  } else {
    return fail(FFK_ERR_UNSUPPORTED, "gemm: dtype %d not supported", dtype);
  }
  FFK_HIP(e);
  return FFK_OK;
}

}  // namespace ffk

using namespace ffk;

extern "C" int ffk_gemm_kernel_name(int dtype, int trans_a, int trans_b, int64_t M, int64_t N, int64_t K,
                                    int has_bias, int activation, char *name, size_t name_bytes) {
  FFK_REQUIRE(name != nullptr && name_bytes > 0, "gemm_kernel_name: no room for the name");
  FFK_REQUIRE(M > 0 && N > 0 && K > 0, "gemm_kernel_name: non-positive dimension");
  name[0] = 0;
  // dense, 16-byte aligned operands: the addresses only have to pass the alignment checks,
  // nothing is launched while the sink is set
  void *const somewhere = reinterpret_cast<void *>(uintptr_t(1) << 20);
  GemmEpilogue ep;
  ep.bias = has_bias ? somewhere : nullptr;
  ep.activation = activation;
  tl_name_sink = name;
  tl_name_sink_bytes = name_bytes;
  int const rc = gemm_dispatch(nullptr, dtype, trans_a != 0, trans_b != 0, M, N, K, somewhere, trans_a ? M : K,
                               somewhere, trans_b ? K : N, somewhere, N, ep);
  tl_name_sink = nullptr;
  tl_name_sink_bytes = 0;
  return rc;
}

extern "C" int ffk_gemm(ffk_stream_t stream, int dtype, int trans_a,
                        int trans_b, int64_t M, int64_t N, int64_t K,
                        void const *A, void const *B, void *C, int accumulate) {
  GemmEpilogue ep;
  ep.accumulate = accumulate != 0;
  return gemm_dispatch(as_stream(stream), dtype, trans_a != 0, trans_b != 0, M,
                       N, K, A, trans_a ? M : K, B, trans_b ? K : N, C, N, ep);
}
