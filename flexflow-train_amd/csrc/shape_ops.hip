// Transpose and Gather for gfx950 (reference: lib/kernels/src/cuda/ops/
// transpose_kernels.cu:27-110 and gather_kernels.cu:23-190).
//
// Transpose: output dim i is input dim perm[i] (dims in FF order, dim 0
// outermost).  The reference walks every output element through a
// divide/modulo chain and reads the input with whatever stride falls out
// (transpose_simple_kernel).  Here the permutation is first simplified on the
// host (dims of extent 1 dropped, dims that stay neighbours merged) and then
// one of three kernels runs:
//   * nothing moves           -> a flat copy / add;
//   * the last dim stays last -> rows are copied whole, 16 bytes per lane;
//   * the last dim changes    -> 64 x 64 tiles go through LDS so that both the
//     reads (along the input's last dim) and the writes (along the output's)
//     are contiguous.
// Backward is the inverse permutation of the output gradient, added to or
// stored into the input gradient.  (The reference's kernel computes
// `out += out * beta + in` in both directions, i.e. it adds into memory the
// forward never initialised and doubles the old gradient in backward; the
// intended `out = in` / `in_grad += out_grad` is what runs here.)
//
// Gather (torch.gather along one dim): with tensors viewed as
// [outer, dim_size, stride], output[o, j, s] = input[o, index[o, j, s], s].
// Backward scatters with hardware fp32 atomics like the reference.
#include "ffk_common.h"
#include <type_traits>

namespace ffk {

constexpr int kMaxDims = 8;
constexpr int kShapeThreads = 256;
constexpr int kTile = 64;

struct PermuteArgs {
  int nd;                       // simplified rank
  int64_t out_dim[kMaxDims];    // output extents
  int64_t in_stride[kMaxDims];  // input stride (elements) of the dim that lands at output position i
};

enum AddMode { kStore = 0, kAddF32 = 1, kAddBf16 = 2 };

template <typename U, int MODE>
__device__ __forceinline__ void put(U *dst, U v) {
  if constexpr (MODE == kStore) {
    *dst = v;
  } else if constexpr (MODE == kAddF32) {
    float const a = __builtin_bit_cast(float, *dst), b = __builtin_bit_cast(float, v);
    *dst = __builtin_bit_cast(U, a + b);
  } else {
    float const a = bf16_bits_to_f32(*dst), b = bf16_bits_to_f32(v);
    *dst = (U)f32_to_bf16_bits(a + b);
  }
}

// Divisions by the row length and by the outer output extents as multiplications (a 64-bit
// division by a kernel argument is some 130 instructions, and a unit needs one per outer dim).
struct PermuteDivs {
  FastDiv by_units;
  FastDiv by_dim[kMaxDims];
};

// 32-bit indices while index + one grid stride cannot wrap
static inline bool fits_fast_index(int64_t total, int64_t threads_per_block) {
  return total < ((int64_t)1 << 31) - (int64_t)kNumCU * 64 * threads_per_block;
}

// The last dim stays last: one unit (an element, or a 16-byte piece of a row)
// per lane; its row is decomposed over the outer output dims.  BIG: 64-bit unit indices.
template <typename U, int MODE, int EPU /* elements per unit, for the typed add */, typename E, bool BIG>
__global__ __launch_bounds__(kShapeThreads) void permute_rows_kernel(U const *__restrict__ in, U *out, PermuteArgs a,
                                                                      int64_t units_per_row, int64_t total_units,
                                                                      PermuteDivs dv) {
  using index_t = std::conditional_t<BIG, int64_t, uint32_t>;
  index_t const stride = (index_t)gridDim.x * kShapeThreads;
  for (index_t q = (index_t)blockIdx.x * kShapeThreads + threadIdx.x; q < (index_t)total_units; q += stride) {
    int64_t in_row = 0;  // in units of elements
    int64_t cu;
    if constexpr (BIG) {
      int64_t row = q / units_per_row;
      cu = q - row * units_per_row;
#pragma unroll 1
      for (int i = a.nd - 2; i >= 0; i--) {
        int64_t const r = row / a.out_dim[i];
        in_row += (row - r * a.out_dim[i]) * a.in_stride[i];
        row = r;
      }
    } else {
      uint32_t row, c;
      dv.by_units.divmod(q, row, c);
      cu = c;
#pragma unroll 1
      for (int i = a.nd - 2; i >= 0; i--) {
        uint32_t r, rem;
        dv.by_dim[i].divmod(row, r, rem);
        in_row += (int64_t)rem * a.in_stride[i];
        row = r;
      }
    }
    U const v = in[in_row / EPU + cu];
    if constexpr (MODE == kStore) {
      out[q] = v;
    } else {
      // typed add, element by element inside the unit
      U o = out[q];
      E *oe = reinterpret_cast<E *>(&o);
      E const *ve = reinterpret_cast<E const *>(&v);
#pragma unroll
      for (int e = 0; e < EPU; e++) put<E, MODE>(oe + e, ve[e]);
      out[q] = o;
    }
  }
}

// The last dim changes: tiles of kTile (input's last dim, "a") x kTile (the
// input dim that becomes the output's last, "b").  blockIdx.x walks a,
// blockIdx.y walks b, blockIdx.z (and a loop) the remaining output dims.
struct TileArgs {
  int n_outer;
  int64_t outer_dim[kMaxDims], outer_in_stride[kMaxDims], outer_out_stride[kMaxDims];
  int64_t A, B;           // extents of a and b
  int64_t in_stride_b;    // input stride of b (a's is 1)
  int64_t out_stride_a;   // output stride of a (b's is 1)
  int64_t outer_total;
};

template <typename E, int MODE>
__global__ __launch_bounds__(kShapeThreads) void permute_tiles_kernel(E const *__restrict__ in, E *out, TileArgs t) {
  __shared__ E tile[kTile][kTile + 1];
  int const tx = threadIdx.x & (kTile - 1), ty = threadIdx.x / kTile;  // ty in [0, 4)
  int64_t const a0 = (int64_t)blockIdx.x * kTile, b0 = (int64_t)blockIdx.y * kTile;
  for (int64_t o = blockIdx.z; o < t.outer_total; o += gridDim.z) {
    int64_t rest = o, in_off = 0, out_off = 0;
#pragma unroll 1
    for (int i = t.n_outer - 1; i >= 0; i--) {
      int64_t const r = rest / t.outer_dim[i];
      int64_t const c = rest - r * t.outer_dim[i];
      in_off += c * t.outer_in_stride[i];
      out_off += c * t.outer_out_stride[i];
      rest = r;
    }
#pragma unroll
    for (int k = 0; k < kTile; k += kShapeThreads / kTile) {
      int64_t const bb = b0 + ty + k, aa = a0 + tx;
      if (bb < t.B && aa < t.A) tile[ty + k][tx] = in[in_off + bb * t.in_stride_b + aa];
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < kTile; k += kShapeThreads / kTile) {
      int64_t const aa = a0 + ty + k, bb = b0 + tx;
      if (aa < t.A && bb < t.B) put<E, MODE>(out + out_off + aa * t.out_stride_a + bb, tile[tx][ty + k]);
    }
    __syncthreads();
  }
}

// The same tiles moved in 16-byte pieces on both sides: a lane fetches V
// consecutive a of one b, and later stores V consecutive b of one a, picking
// them out of V rows of the staged tile.  Needs A, B, both strides and every
// outer stride a multiple of V and 16-byte aligned tensors; one-element
// transactions (128 bytes per wave for bf16) otherwise leave the bf16
// transpose at under half of what the wide form moves.
// STREAM: a tensor too large to stay in the last-level cache is read past the caches (its stores stay
// ordinary: the strided 256-byte row pieces of a tile want the L2's write combining; streaming them too
// cost 10%).
template <typename E, int MODE, bool STREAM>
__global__ __launch_bounds__(kShapeThreads) void permute_tiles_wide_kernel(E const *__restrict__ in, E *out, TileArgs t) {
  constexpr int V = 16 / (int)sizeof(E);
  // Row pitch of the staged tile.  4-byte elements: an odd pitch, so that the column reads of the
  // second phase (pieces 4 rows apart, 4 output rows per wave) fall into distinct banks; the first
  // phase then stores its piece as 4 words.  Other sizes: rows stay 16-byte aligned.
  constexpr bool kOddPitch = sizeof(E) == 4;
  constexpr int S = kOddPitch ? kTile + 1 : kTile + V;
  constexpr int CPR = kTile / V;         // 16-byte pieces per tile row
  constexpr int RPP = kShapeThreads / CPR;  // tile rows per pass
  __shared__ __attribute__((aligned(16))) E tile[kTile * S];
  int const piece = threadIdx.x % CPR, row = threadIdx.x / CPR;
  int64_t const a0 = (int64_t)blockIdx.x * kTile, b0 = (int64_t)blockIdx.y * kTile;
  for (int64_t o = blockIdx.z; o < t.outer_total; o += gridDim.z) {
    int64_t rest = o, in_off = 0, out_off = 0;
#pragma unroll 1
    for (int i = t.n_outer - 1; i >= 0; i--) {
      int64_t const r = rest / t.outer_dim[i];
      int64_t const c = rest - r * t.outer_dim[i];
      in_off += c * t.outer_in_stride[i];
      out_off += c * t.outer_out_stride[i];
      rest = r;
    }
#pragma unroll
    for (int k = 0; k < kTile; k += RPP) {
      int64_t const bb = b0 + row + k, aa = a0 + piece * V;
      if (bb < t.B && aa < t.A) {  // A and B are multiples of V: a piece is inside or outside as a whole
        u32x4 const *const src = reinterpret_cast<u32x4 const *>(in + in_off + bb * t.in_stride_b + aa);
        u32x4 const q = STREAM ? __builtin_nontemporal_load(src) : *src;
        if constexpr (kOddPitch) {
#pragma unroll
          for (int e = 0; e < V; e++) tile[(row + k) * S + piece * V + e] = (E)q[e];
        } else {
          *reinterpret_cast<u32x4 *>(tile + (row + k) * S + piece * V) = q;
        }
      }
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < kTile; k += RPP) {
      int64_t const aa = a0 + row + k, bb = b0 + piece * V;
      if (aa < t.A && bb < t.B) {
        union {
          u32x4 q;
          E e[V];
        } v;
#pragma unroll
        for (int e = 0; e < V; e++) v.e[e] = tile[(piece * V + e) * S + row + k];
        E *dst = out + out_off + aa * t.out_stride_a + bb;
        if constexpr (MODE != kStore) {
          union {
            u32x4 q;
            E e[V];
          } old;
          old.q = *reinterpret_cast<u32x4 const *>(dst);
#pragma unroll
          for (int e = 0; e < V; e++) put<E, MODE>(&old.e[e], v.e[e]);
          v.q = old.q;
        }
        *reinterpret_cast<u32x4 *>(dst) = v.q;
      }
    }
    __syncthreads();
  }
}

template <typename U, int MODE, typename E>
__global__ __launch_bounds__(kShapeThreads) void flat_move_kernel(U const *__restrict__ in, U *out, int64_t units) {
  constexpr int EPU = sizeof(U) / sizeof(E);
  int64_t const stride = (int64_t)gridDim.x * kShapeThreads;
  for (int64_t q = (int64_t)blockIdx.x * kShapeThreads + threadIdx.x; q < units; q += stride) {
    U const v = in[q];
    if constexpr (MODE == kStore) {
      out[q] = v;
    } else {
      U o = out[q];
      E *oe = reinterpret_cast<E *>(&o);
      E const *ve = reinterpret_cast<E const *>(&v);
#pragma unroll
      for (int e = 0; e < EPU; e++) put<E, MODE>(oe + e, ve[e]);
      out[q] = o;
    }
  }
}

static unsigned blocks_for(int64_t units) {
  int64_t b = ceil_div(units > 0 ? units : 1, kShapeThreads);
  int64_t const cap = (int64_t)kNumCU * 32;
  return (unsigned)(b < cap ? b : cap);
}

// E: element storage type (uint16_t / uint32_t / uint64_t / uint8_t)
template <typename E, int MODE>
static hipError_t permute_typed(hipStream_t st, void const *in, void *out, int nd, int64_t const *in_dim,
                                int const *perm) {
  // simplified problem: od[i] = extent of output dim i, is[i] = input stride of that dim
  int64_t in_stride_full[kMaxDims];
  {
    int64_t s = 1;
    for (int i = nd - 1; i >= 0; i--) {
      in_stride_full[i] = s;
      s *= in_dim[i];
    }
  }
  int64_t od[kMaxDims], is[kMaxDims];
  int n = 0;
  for (int i = 0; i < nd; i++) {
    int64_t const ext = in_dim[perm[i]];
    if (ext == 1) continue;  // contributes nothing to any offset
    if (n > 0 && is[n - 1] == ext * in_stride_full[perm[i]]) {
      // this dim directly follows the previous one in the input too: one dim
      od[n - 1] *= ext;
      is[n - 1] = in_stride_full[perm[i]];
    } else {
      od[n] = ext;
      is[n] = in_stride_full[perm[i]];
      n++;
    }
  }
  int64_t total = 1;
  for (int i = 0; i < n; i++) total *= od[i];
  if (total == 0) return hipSuccess;
  bool const wide_ok = reinterpret_cast<uintptr_t>(in) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0;
  constexpr int VE = 16 / (int)sizeof(E);  // elements per 16-byte unit
  if (n <= 1) {
    // nothing moves
    if (wide_ok && total % VE == 0) {
      flat_move_kernel<u32x4, MODE, E><<<blocks_for(total / VE), kShapeThreads, 0, st>>>(
          static_cast<u32x4 const *>(in), static_cast<u32x4 *>(out), total / VE);
    } else {
      flat_move_kernel<E, MODE, E><<<blocks_for(total), kShapeThreads, 0, st>>>(
          static_cast<E const *>(in), static_cast<E *>(out), total);
    }
    return hipGetLastError();
  }
  if (is[n - 1] == 1) {
    // rows stay rows
    PermuteArgs a;
    a.nd = n;
    for (int i = 0; i < n; i++) {
      a.out_dim[i] = od[i];
      a.in_stride[i] = is[i];
    }
    int64_t const L = od[n - 1];
    bool wide = wide_ok && L % VE == 0;
    for (int i = 0; i < n - 1; i++) wide = wide && is[i] % VE == 0;
    int64_t const units_per_row = wide ? L / VE : L, units = wide ? total / VE : total;
    bool const fast = fits_fast_index(units, kShapeThreads);
    PermuteDivs dv{};
    if (fast) {
      dv.by_units = make_fast_div((uint32_t)units_per_row);
      for (int i = 0; i < n - 1; i++) dv.by_dim[i] = make_fast_div((uint32_t)od[i]);
    }
#define FFK_PERMUTE_ROWS(U_, EPU_, BIG_)                                                                   \
  permute_rows_kernel<U_, MODE, EPU_, E, BIG_><<<blocks_for(units), kShapeThreads, 0, st>>>(               \
      static_cast<U_ const *>(in), static_cast<U_ *>(out), a, units_per_row, units, dv)
    if (wide) {
      if (fast) FFK_PERMUTE_ROWS(u32x4, VE, false);
      else FFK_PERMUTE_ROWS(u32x4, VE, true);
    } else {
      if (fast) FFK_PERMUTE_ROWS(E, 1, false);
      else FFK_PERMUTE_ROWS(E, 1, true);
    }
#undef FFK_PERMUTE_ROWS
    return hipGetLastError();
  }
  // tiles: a = the output position whose input stride is 1, b = the last output position
  int pa = -1;
  for (int i = 0; i < n; i++) {
    if (is[i] == 1) pa = i;
  }
  if (pa < 0) return hipErrorInvalidValue;  // cannot happen: some dim has input stride 1
  int64_t out_stride[kMaxDims];
  {
    int64_t s = 1;
    for (int i = n - 1; i >= 0; i--) {
      out_stride[i] = s;
      s *= od[i];
    }
  }
  TileArgs t;
  t.n_outer = 0;
  t.outer_total = 1;
  for (int i = 0; i < n - 1; i++) {
    if (i == pa) continue;
    t.outer_dim[t.n_outer] = od[i];
    t.outer_in_stride[t.n_outer] = is[i];
    t.outer_out_stride[t.n_outer] = out_stride[i];
    t.outer_total *= od[i];
    t.n_outer++;
  }
  t.A = od[pa];
  t.B = od[n - 1];
  t.in_stride_b = is[n - 1];
  t.out_stride_a = out_stride[pa];
  int64_t const gx = ceil_div(t.A, kTile), gy = ceil_div(t.B, kTile);
  if (gx > 0x7fffffff || gy > 65535) return hipErrorInvalidValue;
  int64_t gz = t.outer_total < 65535 ? t.outer_total : 65535;
  bool wide_tiles = wide_ok && sizeof(E) >= 2 && t.A % VE == 0 && t.B % VE == 0 && t.in_stride_b % VE == 0 &&
                    t.out_stride_a % VE == 0;
  for (int i = 0; i < t.n_outer; i++) {
    wide_tiles = wide_tiles && t.outer_in_stride[i] % VE == 0 && t.outer_out_stride[i] % VE == 0;
  }
  if (wide_tiles && MODE == kStore && stream_past_caches(total, sizeof(E))) {
    permute_tiles_wide_kernel<E, MODE, true><<<dim3((unsigned)gx, (unsigned)gy, (unsigned)gz), kShapeThreads, 0, st>>>(
        static_cast<E const *>(in), static_cast<E *>(out), t);
  } else if (wide_tiles) {
    permute_tiles_wide_kernel<E, MODE, false><<<dim3((unsigned)gx, (unsigned)gy, (unsigned)gz), kShapeThreads, 0, st>>>(
        static_cast<E const *>(in), static_cast<E *>(out), t);
  } else {
    permute_tiles_kernel<E, MODE><<<dim3((unsigned)gx, (unsigned)gy, (unsigned)gz), kShapeThreads, 0, st>>>(
        static_cast<E const *>(in), static_cast<E *>(out), t);
  }
  return hipGetLastError();
}

static int permute_any(char const *who, ffk_stream_t stream, int dtype, void const *in, void *out, int nd,
                       int64_t const *in_dim, int const *perm, int accumulate) {
  FFK_REQUIRE(nd >= 1 && nd <= kMaxDims, "%s: 1 to %d dims supported, got %d", who, kMaxDims, nd);
  FFK_REQUIRE(in_dim != nullptr && perm != nullptr, "%s: NULL argument", who);
  bool seen[kMaxDims] = {};
  int64_t total = 1;
  for (int i = 0; i < nd; i++) {
    FFK_REQUIRE(perm[i] >= 0 && perm[i] < nd && !seen[perm[i]], "%s: not a permutation", who);
    seen[perm[i]] = true;
    FFK_REQUIRE(in_dim[i] >= 0, "%s: negative extent", who);
    total *= in_dim[i];
  }
  if (total == 0) return FFK_OK;
  FFK_REQUIRE(in != nullptr && out != nullptr, "%s: NULL tensor", who);
  FFK_REQUIRE(in != out, "%s: in place is not supported", who);
  hipStream_t st = as_stream(stream);
  hipError_t e;
  if (accumulate) {
    if (dtype == FFK_FLOAT) e = permute_typed<uint32_t, kAddF32>(st, in, out, nd, in_dim, perm);
    else if (dtype == FFK_BF16) e = permute_typed<uint16_t, kAddBf16>(st, in, out, nd, in_dim, perm);
    else return fail(FFK_ERR_UNSUPPORTED, "%s: adding supports float and bf16 (got data type %d)", who, dtype);
  } else {
    switch (dtype) {
      case FFK_BOOL: e = permute_typed<uint8_t, kStore>(st, in, out, nd, in_dim, perm); break;
      case FFK_HALF: case FFK_BF16: e = permute_typed<uint16_t, kStore>(st, in, out, nd, in_dim, perm); break;
      case FFK_INT32: case FFK_FLOAT: e = permute_typed<uint32_t, kStore>(st, in, out, nd, in_dim, perm); break;
      case FFK_INT64: case FFK_DOUBLE: e = permute_typed<uint64_t, kStore>(st, in, out, nd, in_dim, perm); break;
      default: return fail(FFK_ERR_UNSUPPORTED, "%s: data type %d not supported", who, dtype);
    }
  }
  FFK_HIP(e);
  return FFK_OK;
}

// ---- gather -------------------------------------------------------------------

// One output element per lane.  BIG: 64-bit element indices; otherwise 32-bit with the two
// divisions as multiplications.
struct GatherDivs {
  FastDiv by_out_plane, by_stride;
};

template <bool BIG, typename index_t>
__device__ __forceinline__ void gather_split(index_t o, int64_t out_plane, int64_t stride, GatherDivs const &dv,
                                             int64_t &outer, int64_t &left) {
  if constexpr (BIG) {
    outer = o / out_plane;
    left = o % stride;
  } else {
    uint32_t q, r;
    dv.by_stride.divmod(o, q, r);
    left = r;
    outer = dv.by_out_plane.div(o);
  }
}

template <typename E, typename IT, bool BIG>
__global__ __launch_bounds__(kShapeThreads) void gather_fwd_kernel(E const *__restrict__ in, IT const *__restrict__ index,
                                                                    E *__restrict__ out, int64_t total, int64_t stride,
                                                                    int64_t in_dim, int64_t out_dim, GatherDivs dv) {
  using index_t = std::conditional_t<BIG, int64_t, uint32_t>;
  index_t const step = (index_t)gridDim.x * kShapeThreads;
  int64_t const out_plane = stride * out_dim, in_plane = stride * in_dim;
  for (index_t o = (index_t)blockIdx.x * kShapeThreads + threadIdx.x; o < (index_t)total; o += step) {
    int64_t outer, left;
    gather_split<BIG>(o, out_plane, stride, dv, outer, left);
    int64_t const j = (int64_t)index[o];
    // an index outside the dim reads nothing (the reference would read out of bounds)
    out[o] = (j >= 0 && j < in_dim) ? in[outer * in_plane + j * stride + left] : E(0);
  }
}

template <typename IT, bool BIG>
__global__ __launch_bounds__(kShapeThreads) void gather_bwd_kernel(float const *__restrict__ dout,
                                                                    IT const *__restrict__ index, float *din,
                                                                    int64_t total, int64_t stride, int64_t in_dim,
                                                                    int64_t out_dim, GatherDivs dv) {
  using index_t = std::conditional_t<BIG, int64_t, uint32_t>;
  index_t const step = (index_t)gridDim.x * kShapeThreads;
  int64_t const out_plane = stride * out_dim, in_plane = stride * in_dim;
  for (index_t o = (index_t)blockIdx.x * kShapeThreads + threadIdx.x; o < (index_t)total; o += step) {
    int64_t outer, left;
    gather_split<BIG>(o, out_plane, stride, dv, outer, left);
    int64_t const j = (int64_t)index[o];
    if (j >= 0 && j < in_dim) atomicAdd(din + outer * in_plane + j * stride + left, dout[o]);
  }
}

// Gather along the last dim when most of a row is picked: a workgroup stages its row in LDS with
// 16-byte loads and picks from there.  Picking from memory fetches a 128-byte line per lane for
// one element, and a row's lines again for every pick that lands in them.
constexpr int kGatherRowBytes = 64 * 1024;  // staged row, at most (two workgroups per CU)

template <typename E, typename IT>
__global__ __launch_bounds__(kShapeThreads) void gather_rows_lds_kernel(E const *__restrict__ in, IT const *__restrict__ index,
                                                                         E *__restrict__ out, int64_t in_dim, int64_t out_dim) {
  extern __shared__ __attribute__((aligned(16))) unsigned char gather_row[];
  E *const row = reinterpret_cast<E *>(gather_row);
  int64_t const r = blockIdx.x;
  E const *const src = in + r * in_dim;
  constexpr int V = 16 / (int)sizeof(E);
  if (in_dim % V == 0 && reinterpret_cast<uintptr_t>(src) % 16 == 0) {
    for (int64_t c = threadIdx.x; c < in_dim / V; c += kShapeThreads) {
      reinterpret_cast<u32x4 *>(row)[c] = reinterpret_cast<u32x4 const *>(src)[c];
    }
  } else {
    for (int64_t c = threadIdx.x; c < in_dim; c += kShapeThreads) row[c] = src[c];
  }
  __syncthreads();
  for (int64_t o = threadIdx.x; o < out_dim; o += kShapeThreads) {
    int64_t const j = (int64_t)index[r * out_dim + o];
    // an index outside the dim reads nothing (the reference would read out of bounds)
    out[r * out_dim + o] = (j >= 0 && j < in_dim) ? row[j] : E(0);
  }
}

// The backward of such a Gather: the workgroup sums its row's gradient in LDS (LDS float adds: no
// trip to memory per element, no contention between rows) and adds the touched elements to the
// input gradient once, 16 bytes per lane where the row allows.  Adds through memory atomics run at
// a few per cent of the memory rate.
template <typename IT>
__global__ __launch_bounds__(kShapeThreads) void gather_rows_lds_bwd_kernel(float const *__restrict__ dout,
                                                                             IT const *__restrict__ index, float *din,
                                                                             int64_t in_dim, int64_t out_dim) {
  extern __shared__ __attribute__((aligned(16))) unsigned char gather_row[];
  float *const row = reinterpret_cast<float *>(gather_row);
  int64_t const r = blockIdx.x;
  float *const dst = din + r * in_dim;
  bool const wide = in_dim % 4 == 0 && reinterpret_cast<uintptr_t>(dst) % 16 == 0;
  // whole 16-byte groups are cleared (the LDS size is rounded up to them)
  for (int64_t c = threadIdx.x; c < (in_dim + 3) / 4; c += kShapeThreads) {
    reinterpret_cast<f32x4 *>(row)[c] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  __syncthreads();
  for (int64_t o = threadIdx.x; o < out_dim; o += kShapeThreads) {
    int64_t const j = (int64_t)index[r * out_dim + o];
    if (j >= 0 && j < in_dim) atomicAdd(row + j, dout[r * out_dim + o]);
  }
  __syncthreads();
  // an element nobody picked keeps its bits (the reference's atomics never touch it)
  if (wide) {
    for (int64_t c = threadIdx.x; c < in_dim / 4; c += kShapeThreads) {
      f32x4 const v = reinterpret_cast<f32x4 const *>(row)[c];
      if (v[0] != 0.f || v[1] != 0.f || v[2] != 0.f || v[3] != 0.f) {
        f32x4 d = reinterpret_cast<f32x4 const *>(dst)[c];
        for (int e = 0; e < 4; ++e) d[e] = v[e] != 0.f ? d[e] + v[e] : d[e];
        reinterpret_cast<f32x4 *>(dst)[c] = d;
      }
    }
  } else {
    for (int64_t c = threadIdx.x; c < in_dim; c += kShapeThreads) {
      float const v = row[c];
      if (v != 0.f) dst[c] += v;
    }
  }
}

// the divisors of a gather over `total` output elements, or false when 32-bit indices do not fit
static bool gather_divs(int64_t total, int64_t stride, int64_t out_dim, GatherDivs &dv) {
  if (!fits_fast_index(total, kShapeThreads) || total == 0) return false;
  // total = outer * out_plane < 2^31, so both divisors are below 2^31
  dv.by_out_plane = make_fast_div((uint32_t)(stride * out_dim));
  dv.by_stride = make_fast_div((uint32_t)stride);
  return true;
}

}  // namespace ffk

using namespace ffk;

extern "C" int ffk_transpose_forward(ffk_stream_t stream, int dtype, void const *input, void *output, int num_dims,
                                     int64_t const *input_dims, int const *perm) {
  return permute_any("transpose_forward", stream, dtype, input, output, num_dims, input_dims, perm, 0);
}

extern "C" int ffk_transpose_backward(ffk_stream_t stream, int dtype, void const *output_grad, void *input_grad,
                                      int num_dims, int64_t const *input_dims, int const *perm, int accumulate) {
  FFK_REQUIRE(num_dims >= 1 && num_dims <= kMaxDims && input_dims && perm, "transpose_backward: bad arguments");
  // the output gradient has dims input_dims[perm[i]]; moving it back is the inverse permutation
  int64_t out_dims[kMaxDims];
  int inverse[kMaxDims];
  for (int i = 0; i < num_dims; i++) {
    FFK_REQUIRE(perm[i] >= 0 && perm[i] < num_dims, "transpose_backward: not a permutation");
    out_dims[i] = input_dims[perm[i]];
    inverse[perm[i]] = i;
  }
  return permute_any("transpose_backward", stream, dtype, output_grad, input_grad, num_dims, out_dims, inverse,
                     accumulate);
}

extern "C" int ffk_gather_forward(ffk_stream_t stream, int dtype, int index_dtype, void const *input,
                                  void const *index, void *output, int64_t outer, int64_t input_dim_size,
                                  int64_t output_dim_size, int64_t stride) {
  FFK_REQUIRE(outer >= 0 && input_dim_size > 0 && output_dim_size >= 0 && stride > 0, "gather_forward: bad shape");
  FFK_REQUIRE(index_dtype == FFK_INT32 || index_dtype == FFK_INT64, "gather_forward: index must be int32 or int64");
  int64_t const total = outer * output_dim_size * stride;
  if (total == 0) return FFK_OK;
  FFK_REQUIRE(input && index && output, "gather_forward: NULL tensor");
  hipStream_t st = as_stream(stream);
  unsigned const blocks = blocks_for(total);
  // last-dim gather that picks at least an eighth of a row that fits LDS: stage the row
  bool const staged = stride == 1 && output_dim_size * 8 >= input_dim_size && outer < (int64_t(1) << 31) &&
                      input_dim_size * (int64_t)dtype_size(dtype) <= kGatherRowBytes;
#define FFK_GATHER_STAGED(E, IT)                                                                             \
  gather_rows_lds_kernel<E, IT><<<(unsigned)outer, kShapeThreads, (size_t)(input_dim_size * sizeof(E) + 15) / 16 * 16, st>>>( \
      static_cast<E const *>(input), static_cast<IT const *>(index), static_cast<E *>(output), input_dim_size, \
      output_dim_size)
  GatherDivs dv{};
  bool const fast = gather_divs(total, stride, output_dim_size, dv);
#define FFK_GATHER_ONE(E, IT, BIG)                                                                           \
  gather_fwd_kernel<E, IT, BIG><<<blocks, kShapeThreads, 0, st>>>(                                           \
      static_cast<E const *>(input), static_cast<IT const *>(index), static_cast<E *>(output), total, stride, \
      input_dim_size, output_dim_size, dv)
#define FFK_GATHER(E)                                                                                        \
  do {                                                                                                       \
    if (staged) {                                                                                            \
      if (index_dtype == FFK_INT32) FFK_GATHER_STAGED(E, int32_t);                                           \
      else FFK_GATHER_STAGED(E, int64_t);                                                                    \
    } else if (index_dtype == FFK_INT32) {                                                                   \
      if (fast) FFK_GATHER_ONE(E, int32_t, false);                                                           \
      else FFK_GATHER_ONE(E, int32_t, true);                                                                 \
    } else {                                                                                                 \
      if (fast) FFK_GATHER_ONE(E, int64_t, false);                                                           \
      else FFK_GATHER_ONE(E, int64_t, true);                                                                 \
    }                                                                                                        \
  } while (0)
  switch (dtype) {
    case FFK_BOOL: FFK_GATHER(uint8_t); break;
    case FFK_HALF: case FFK_BF16: FFK_GATHER(uint16_t); break;
    case FFK_INT32: case FFK_FLOAT: FFK_GATHER(uint32_t); break;
    case FFK_INT64: case FFK_DOUBLE: FFK_GATHER(uint64_t); break;
    default: return fail(FFK_ERR_UNSUPPORTED, "gather_forward: data type %d not supported", dtype);
  }
#undef FFK_GATHER
#undef FFK_GATHER_ONE
#undef FFK_GATHER_STAGED
  FFK_CHECK_LAUNCH();
  return FFK_OK;
}

extern "C" int ffk_gather_backward(ffk_stream_t stream, int index_dtype, float const *output_grad,
                                   void const *index, float *input_grad, int64_t outer, int64_t input_dim_size,
                                   int64_t output_dim_size, int64_t stride) {
  FFK_REQUIRE(outer >= 0 && input_dim_size > 0 && output_dim_size >= 0 && stride > 0, "gather_backward: bad shape");
  FFK_REQUIRE(index_dtype == FFK_INT32 || index_dtype == FFK_INT64, "gather_backward: index must be int32 or int64");
  int64_t const total = outer * output_dim_size * stride;
  if (total == 0) return FFK_OK;
  FFK_REQUIRE(output_grad && index && input_grad, "gather_backward: NULL tensor");
  hipStream_t st = as_stream(stream);
  unsigned const blocks = blocks_for(total);
  // along the last dim, rows that fit LDS and are picked from at least once per 16 elements
  if (stride == 1 && output_dim_size * 16 >= input_dim_size && outer < (int64_t(1) << 31) &&
      input_dim_size * (int64_t)sizeof(float) <= kGatherRowBytes) {
    size_t const lds = (size_t)(input_dim_size + 3) / 4 * 16;
    if (index_dtype == FFK_INT32) {
      gather_rows_lds_bwd_kernel<int32_t><<<(unsigned)outer, kShapeThreads, lds, st>>>(
          output_grad, static_cast<int32_t const *>(index), input_grad, input_dim_size, output_dim_size);
    } else {
      gather_rows_lds_bwd_kernel<int64_t><<<(unsigned)outer, kShapeThreads, lds, st>>>(
          output_grad, static_cast<int64_t const *>(index), input_grad, input_dim_size, output_dim_size);
    }
    FFK_CHECK_LAUNCH();
    return FFK_OK;
  }
  GatherDivs dv{};
  bool const fast = gather_divs(total, stride, output_dim_size, dv);
#define FFK_GATHER_BWD(IT, BIG)                                                                              \
  gather_bwd_kernel<IT, BIG><<<blocks, kShapeThreads, 0, st>>>(output_grad, static_cast<IT const *>(index), \
                                                               input_grad, total, stride, input_dim_size,   \
                                                               output_dim_size, dv)
  if (index_dtype == FFK_INT32) {
    if (fast) FFK_GATHER_BWD(int32_t, false);
    else FFK_GATHER_BWD(int32_t, true);
  } else {
    if (fast) FFK_GATHER_BWD(int64_t, false);
    else FFK_GATHER_BWD(int64_t, true);
  }
#undef FFK_GATHER_BWD
  FFK_CHECK_LAUNCH();
  return FFK_OK;
}
