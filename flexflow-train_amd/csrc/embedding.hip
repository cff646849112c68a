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
#include "radix_sort.h"
#include <cstdlib>
#include <type_traits>
#include <cstring>

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
  __builtin_nontemporal_store(u32x2{pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])}, reinterpret_cast<u32x2 *>(p));
}
template <>
__device__ __forceinline__ void store_out<bf16, 8>(bf16 *p, float const (&v)[8]) {
  VecIO<bf16>::store_stream(p, v);
}

// V elements of a table row as floats: 16-byte loads
template <typename WT, int V>
__device__ __forceinline__ void load_row(WT const *p, float (&v)[V]) {
  if constexpr (sizeof(WT) == 4 && V == 8) {
    float a[4], b[4];
    VecIO<float>::load(p, a);
    VecIO<float>::load(p + 4, b);
#pragma unroll
    for (int e = 0; e < 4; e++) {
      v[e] = a[e];
      v[4 + e] = b[e];
    }
  } else {
    static_assert(V == VecIO<WT>::kVec, "one 16-byte load");
    VecIO<WT>::load(p, v);
  }
}
// elements per thread: what makes the store 16 bytes (8 for a bf16 output), at least one 16-byte load
template <typename WT, typename OT>
constexpr int emb_vec() {
  return sizeof(OT) == 2 ? 8 : VecIO<WT>::kVec;
}

// One thread per (bag, 16-byte vector of the row).  BIG: 2^31 and more threads' worth of
// work, 64-bit index arithmetic; otherwise 32-bit with the division by nvec as a multiplication
// (the 64-bit division alone was 130 of the 250 instructions a thread of the plain gather ran,
// and made that kernel bound by the vector ALU).
// CHUNKED: the kernel for bags of eight entries and more (its row buffers cost the plain
// gather half its waves per CU, so single lookups run the instantiation without them).
template <typename IT, typename WT, typename OT, bool BIG, bool CHUNKED>
__global__ __launch_bounds__(kEmbThreads) void embedding_fwd_vec_kernel(
    IT const *__restrict__ idx, OT *__restrict__ out, WT const *__restrict__ W,
    int64_t num_bags, int bag, int nvec, int64_t dim, int64_t num_entries,
    float scale, FastDiv by_nvec) {
  constexpr int V = emb_vec<WT, OT>();
  using index_t = std::conditional_t<BIG, int64_t, uint32_t>;
  index_t const total = (index_t)(num_bags * nvec);
  index_t const stride = (index_t)gridDim.x * kEmbThreads;
  for (index_t i = (index_t)blockIdx.x * kEmbThreads + threadIdx.x; i < total; i += stride) {
    int64_t b;
    int v;
    if constexpr (BIG) {
      b = i / nvec;
      v = (int)(i % nvec);
    } else {
      uint32_t q, r;
      by_nvec.divmod(i, q, r);
      b = q;
      v = (int)r;
    }
    float acc[V];
#pragma unroll
    for (int e = 0; e < V; e++) acc[e] = 0.0f;
    IT const *ib = idx + b * bag;
    int j = 0;
    // Bags of eight entries and more: eight row reads in flight, and the indices of the next
    // eight are asked for before this group's rows are waited for, so a bag of 32 costs one
    // index round trip and four row round trips instead of eight of each.  The sum keeps the
    // order of the entries.
    if constexpr (CHUNKED) {
      constexpr int CH = 8;
      int64_t rn[CH];
#pragma unroll
      for (int u = 0; u < CH; u++) rn[u] = (int64_t)ib[u];
      for (; j + CH <= bag; j += CH) {
        float w[CH][V];
        bool ok[CH];
#pragma unroll
        for (int u = 0; u < CH; u++) {
          ok[u] = (uint64_t)rn[u] < (uint64_t)num_entries;
          load_row<WT, V>(W + (ok[u] ? rn[u] : 0) * dim + (int64_t)v * V, w[u]);
        }
        if (j + 2 * CH <= bag) {
#pragma unroll
          for (int u = 0; u < CH; u++) rn[u] = (int64_t)ib[j + CH + u];
        }
#pragma unroll
        for (int u = 0; u < CH; u++)
#pragma unroll
          for (int e = 0; e < V; e++) acc[e] = acc[e] + (ok[u] ? w[u][e] : 0.0f);
      }
    }
    for (; j + 4 <= bag; j += 4) {  // four row reads in flight
      int64_t r[4];
      float w[4][V];
#pragma unroll
      for (int u = 0; u < 4; u++) r[u] = (int64_t)ib[j + u];
#pragma unroll
      for (int u = 0; u < 4; u++) {
        bool ok = (uint64_t)r[u] < (uint64_t)num_entries;
        load_row<WT, V>(W + (ok ? r[u] : 0) * dim + (int64_t)v * V, w[u]);
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
        load_row<WT, V>(W + r * dim + (int64_t)v * V, w);
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

// HALF and DOUBLE tables (embedding_kernels.cu:374-449,491-566 forward, 609-808 backward): table,
// output and gradients share one type T and all arithmetic is T's own, as in the reference -- a bag
// is summed in T entry by entry, the backward adds T values atomically.  One thread per (bag,
// column); no configuration uses these types, so nothing here is tuned.
template <typename IT, typename T>
__global__ __launch_bounds__(kEmbThreads) void embedding_fwd_typed_kernel(
    IT const *__restrict__ idx, T *__restrict__ out, T const *__restrict__ W,
    int64_t num_bags, int bag, int64_t dim, int64_t num_entries, bool avg) {
  int64_t const total = num_bags * dim;
  int64_t const stride = (int64_t)gridDim.x * kEmbThreads;
  T const scale = (T)(1.0f / (float)bag);  // the reference's `TD scale = 1.0f / in_dim`
  for (int64_t i = (int64_t)blockIdx.x * kEmbThreads + threadIdx.x; i < total; i += stride) {
    int64_t const b = i / dim, d = i % dim;
    T acc = (T)0;
    for (int j = 0; j < bag; j++) {
      int64_t const r = (int64_t)idx[b * bag + j];
      if ((uint64_t)r < (uint64_t)num_entries) acc = acc + W[r * dim + d];
    }
    if (avg) acc = acc * scale;
    out[i] = acc;
  }
}

__device__ __forceinline__ void atomic_add_typed(double *p, double v) { atomicAdd(p, v); }
// no 16-bit atomic: compare-and-swap on the aligned word that holds the half
__device__ __forceinline__ void atomic_add_typed(_Float16 *p, _Float16 v) {
  uintptr_t const a = reinterpret_cast<uintptr_t>(p);
  uint32_t *word = reinterpret_cast<uint32_t *>(a & ~(uintptr_t)3);
  bool const high = (a & 2) != 0;
  uint32_t seen = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  for (;;) {
    uint16_t const bits = high ? (uint16_t)(seen >> 16) : (uint16_t)(seen & 0xffffu);
    _Float16 const sum = __builtin_bit_cast(_Float16, bits) + v;
    uint32_t const sb = __builtin_bit_cast(uint16_t, sum);
    uint32_t const want = high ? (seen & 0x0000ffffu) | (sb << 16) : (seen & 0xffff0000u) | sb;
    uint32_t const prev = atomicCAS(word, seen, want);
    if (prev == seen) break;
    seen = prev;
  }
}

template <typename IT, typename T>
__global__ __launch_bounds__(kEmbThreads) void embedding_bwd_typed_kernel(
    IT const *__restrict__ idx, T const *__restrict__ dY, T *dW,
    int64_t num_bags, int bag, int64_t dim, int64_t num_entries, bool avg) {
  int64_t const total = num_bags * dim;
  int64_t const stride = (int64_t)gridDim.x * kEmbThreads;
  T const scale = (T)(1.0f / (float)bag);
  for (int64_t i = (int64_t)blockIdx.x * kEmbThreads + threadIdx.x; i < total; i += stride) {
    int64_t const b = i / dim, d = i % dim;
    T g = dY[i];
    if (avg) g = g * scale;
    for (int j = 0; j < bag; j++) {
      int64_t const r = (int64_t)idx[b * bag + j];
      if ((uint64_t)r < (uint64_t)num_entries) atomic_add_typed(dW + r * dim + d, g);
    }
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

// Sorted scatter-add.  The atomic kernel above is bound by the rate at which
// the memory side retires fp32 atomics (about 0.7 TB/s of payload measured on
// MI355X, far below HBM).  With scratch from the caller the lookups are sorted
// by row id first (the stable radix sort of radix_sort.h); equal ids then
// form runs, a walker sums the gradient rows of a run in registers and adds the
// sum to the weight-gradient row with ordinary loads and stores, because a run
// that lies inside one walker's chunk is touched by nobody else.  Only runs
// that cross a chunk border (at most two per walker) go through atomics.
constexpr int kEmbChunk = 16;  // sorted positions per walker

template <typename GT>
__device__ __forceinline__ void load_grad4(GT const *p, float (&v)[4]);
template <>
__device__ __forceinline__ void load_grad4<float>(float const *p, float (&v)[4]) {
  f32x4 r = __builtin_nontemporal_load(reinterpret_cast<f32x4 const *>(p));
  v[0] = r[0]; v[1] = r[1]; v[2] = r[2]; v[3] = r[3];
}
template <>
__device__ __forceinline__ void load_grad4<bf16>(bf16 const *p, float (&v)[4]) {
  u32x2 r = __builtin_nontemporal_load(reinterpret_cast<u32x2 const *>(p));
  v[0] = __uint_as_float(r[0] << 16);
  v[1] = __uint_as_float(r[0] & 0xffff0000u);
  v[2] = __uint_as_float(r[1] << 16);
  v[3] = __uint_as_float(r[1] & 0xffff0000u);
}

// LPR lanes share a row, 4 columns per lane and CPL such chunks per lane in
// one pass (columns c = ((k * LPR) + lane) * 4, k < CPL).
// DET: a walker owns every run that STARTS in its chunk and follows it to its
// end, however far; no run is shared, nothing is atomic, and every row is
// summed in ascending lookup order, so the result is bit-reproducible (a very
// popular row is then summed by a single walker, which is slow).
template <typename GT, int LPR, int CPL, bool DET>
__global__ __launch_bounds__(256) void embedding_bwd_sorted_kernel(
    uint32_t const *__restrict__ keys, uint32_t const *__restrict__ vals,
    GT const *__restrict__ dY, float *dW, int64_t n, int bag, int64_t dim,
    uint32_t invalid_key, float scale) {
  int64_t const walker = ((int64_t)blockIdx.x * 256 + threadIdx.x) / LPR;
  int const wl = threadIdx.x % LPR;
  int64_t const p0 = walker * kEmbChunk;
  if (p0 >= n) return;
  int64_t const p1 = min(p0 + (int64_t)kEmbChunk, n);
  int64_t start = p0;
  if (DET) {
    while (start < p1 && start > 0 && keys[start - 1] == keys[start]) start++;
    if (start >= p1) return;
  }
  // is position p part of this walker's work?
  auto mine = [&](int64_t p) {
    return p < p1 || (DET && p < n && keys[p] == keys[p - 1]);
  };
  for (int64_t cbase = 0; cbase < dim; cbase += (int64_t)LPR * 4 * CPL) {
    float acc[CPL][4], cur[CPL][4], nxt[CPL][4];
    auto fetch = [&](int64_t p, float (&v)[CPL][4]) {
      int64_t const l = (int64_t)vals[p];
      GT const *row = dY + (l / bag) * dim;
#pragma unroll
      for (int k = 0; k < CPL; k++) {
        int64_t const c = cbase + ((int64_t)k * LPR + wl) * 4;
        if (c < dim) {
          load_grad4<GT>(row + c, v[k]);
        } else {
          v[k][0] = v[k][1] = v[k][2] = v[k][3] = 0.0f;
        }
      }
    };
#pragma unroll
    for (int k = 0; k < CPL; k++)
#pragma unroll
      for (int e = 0; e < 4; e++) acc[k][e] = 0.0f;
    // a run that began in the previous chunk is shared with that walker
    bool shared_run = !DET && p0 > 0 && keys[p0 - 1] == keys[p0];
    fetch(start, cur);
    for (int64_t p = start; mine(p); p++) {
      bool const more = mine(p + 1);
      if (more) fetch(p + 1, nxt);  // next row in flight while this one is added
      uint32_t const id = keys[p];
#pragma unroll
      for (int k = 0; k < CPL; k++)
#pragma unroll
        for (int e = 0; e < 4; e++) acc[k][e] += cur[k][e];
      bool const run_end = !more || keys[p + 1] != id;
      if (run_end) {
        if (!DET && !more && p + 1 < n && keys[p + 1] == id) shared_run = true;  // continues next door
        if (id != invalid_key) {
#pragma unroll
          for (int k = 0; k < CPL; k++) {
            int64_t const c = cbase + ((int64_t)k * LPR + wl) * 4;
            if (c < dim) {
              float *dst = dW + (int64_t)id * dim + c;
              if (shared_run) {
#pragma unroll
                for (int e = 0; e < 4; e++) atomicAdd(dst + e, acc[k][e] * scale);
              } else {
                f32x4 old = *reinterpret_cast<f32x4 const *>(dst);
                f32x4 upd = {old[0] + acc[k][0] * scale, old[1] + acc[k][1] * scale,
                             old[2] + acc[k][2] * scale, old[3] + acc[k][3] * scale};
                *reinterpret_cast<f32x4 *>(dst) = upd;
              }
            }
          }
        }
        shared_run = false;
#pragma unroll
        for (int k = 0; k < CPL; k++)
#pragma unroll
          for (int e = 0; e < 4; e++) acc[k][e] = 0.0f;
      }
#pragma unroll
      for (int k = 0; k < CPL; k++)
#pragma unroll
        for (int e = 0; e < 4; e++) cur[k][e] = nxt[k][e];
    }
  }
}

// The non-deterministic sorted path: a workgroup of 1024 threads owns
// (1024 / LPR) * kEmbChunk consecutive sorted positions.  Walkers add runs that
// lie inside their chunk straight to memory; the partial sums of runs that
// cross a walker border meet in LDS and are merged by the workgroup, so only
// runs that cross a WORKGROUP border reach memory as atomics.  A row looked up
// thousands of times (Zipf-distributed tokens) then costs one atomic per
// element per workgroup instead of one per walker, which matters because
// atomics to one address are retired one after the other.
constexpr int kEmbBlockThreads = 1024;

// CPL column chunks of 4 per lane and pass (more bytes in flight per walker
// step: the walk is latency-bound otherwise).  LDS: 2 * WPB border partials of
// LPR * 4 * CPL floats, passed as dynamic shared memory.
template <typename GT, int LPR, int CPL>
__global__ __launch_bounds__(kEmbBlockThreads) void embedding_bwd_sorted_block_kernel(
    uint32_t const *__restrict__ keys, uint32_t const *__restrict__ vals,
    GT const *__restrict__ dY, float *dW, int64_t n, int bag, int64_t dim,
    uint32_t invalid_key, float scale) {
  constexpr int WPB = kEmbBlockThreads / LPR;  // walkers per workgroup
  constexpr int PW = LPR * 4 * CPL;            // columns per pass
  extern __shared__ __attribute__((aligned(16))) float emb_part[];  // [2 * WPB][PW]
  __shared__ uint32_t part_id[2 * WPB];
  __shared__ int part_valid[2 * WPB];
  int const w = threadIdx.x / LPR, wl = threadIdx.x % LPR;
  int64_t const block0 = (int64_t)blockIdx.x * WPB * kEmbChunk;
  int64_t const block1 = min(block0 + (int64_t)WPB * kEmbChunk, n);
  int64_t const p0 = block0 + (int64_t)w * kEmbChunk;
  int64_t const p1 = min(p0 + (int64_t)kEmbChunk, n);
  // The walker's 16 (row id, lookup) pairs are fetched once, one pair per lane, and handed round
  // with lane shuffles.  What the walk would otherwise wait for at every position -- the
  // gradient row of the lookup and, where a run ends, the weight-gradient row it is added to --
  // is then asked for two positions ahead.  (Walkers of cold rows, where every position ends a
  // run, set the pace of their workgroup: each of their positions used to cost two dependent
  // memory round trips.)
  int const cnt = (int)max((int64_t)0, min((int64_t)kEmbChunk, n - p0));  // positions that exist
  bool const active = cnt > 0;
  static_assert(LPR >= kEmbChunk, "one pair per lane");
  uint32_t my_key = invalid_key, my_val = 0;
  if (wl < cnt) {
    my_key = keys[p0 + wl];
    my_val = vals[p0 + wl];
    // what the walk needs of a lookup is the gradient row it reads: its bag.  Divided once here,
    // by the lane that holds the pair, not at every position by every lane of the walker.
    if (bag != 1) my_val /= (uint32_t)bag;
  }
  int const wbase = ((threadIdx.x & 63) / LPR) * LPR;  // the walker's first lane in its wave
  uint32_t const key_before = active && p0 > 0 ? keys[p0 - 1] : invalid_key;
  uint32_t const key_after = active && p1 < n ? keys[p1] : invalid_key;
  // every lane of the wave takes part in a shuffle, whatever its walker has to do
  auto key_at = [&](int j) { return (uint32_t)__shfl((int)my_key, wbase + (j < kEmbChunk ? j : kEmbChunk - 1), 64); };
  auto lookup_at = [&](int j) { return (uint32_t)__shfl((int)my_val, wbase + (j < kEmbChunk ? j : kEmbChunk - 1), 64); };
  bool const head_shared = active && p0 > 0 && key_before == key_at(0);
  auto add_row = [&](uint32_t id, int64_t cbase, float const (&acc)[CPL][4], bool atomic) {
#pragma unroll
    for (int k = 0; k < CPL; k++) {
      int64_t const c = cbase + ((int64_t)k * LPR + wl) * 4;
      if (c < dim) {
        float *dst = dW + (int64_t)id * dim + c;
        if (atomic) {
#pragma unroll
          for (int e = 0; e < 4; e++) atomicAdd(dst + e, acc[k][e] * scale);
        } else {
          f32x4 old = *reinterpret_cast<f32x4 const *>(dst);
          f32x4 upd = {old[0] + acc[k][0] * scale, old[1] + acc[k][1] * scale,
                       old[2] + acc[k][2] * scale, old[3] + acc[k][3] * scale};
          *reinterpret_cast<f32x4 *>(dst) = upd;
        }
      }
    }
  };
  for (int64_t cbase = 0; cbase < dim; cbase += PW) {
    if (wl == 0) {
      part_valid[2 * w] = 0;
      part_valid[2 * w + 1] = 0;
    }
    {
      float acc[CPL][4], rows[2][CPL][4];
      f32x4 old[2][CPL];
      // position j's gradient row, and the weight-gradient row of its id if a run of this
      // walker alone ends there (nobody else touches that row during the kernel)
      auto prefetch = [&](int j, uint32_t id, uint32_t next_id, uint32_t l, float (&v)[CPL][4], f32x4 (&o)[CPL]) {
        if (j >= cnt) return;
        GT const *row = dY + (int64_t)l * dim;  // l: the lookup's bag (see my_val)
        bool const ends = j + 1 >= cnt || next_id != id;
#pragma unroll
        for (int k = 0; k < CPL; k++) {
          int64_t const c = cbase + ((int64_t)k * LPR + wl) * 4;
          if (c < dim) {
            load_grad4<GT>(row + c, v[k]);
            if (ends && id != invalid_key) o[k] = *reinterpret_cast<f32x4 const *>(dW + (int64_t)id * dim + c);
          } else {
            v[k][0] = v[k][1] = v[k][2] = v[k][3] = 0.0f;
          }
        }
      };
#pragma unroll
      for (int k = 0; k < CPL; k++)
#pragma unroll
        for (int e = 0; e < 4; e++) acc[k][e] = 0.0f;
      bool shared_run = head_shared;
      // the ids around position j: id_j, id_{j+1}, id_{j+2}, id_{j+3} slide along with j
      uint32_t id0 = key_at(0), id1 = key_at(1), id2 = key_at(2), l0 = lookup_at(0), l1 = lookup_at(1);
      prefetch(0, id0, id1, l0, rows[0], old[0]);
      prefetch(1, id1, id2, l1, rows[1], old[1]);
      auto step = [&](int j, float (&v)[CPL][4], f32x4 (&o)[CPL]) {
        // shuffles first, by every lane
        uint32_t const id3 = key_at(j + 3);
        uint32_t const l2 = lookup_at(j + 2);
        if (j < cnt) {
          uint32_t const id = id0;
#pragma unroll
          for (int k = 0; k < CPL; k++)
#pragma unroll
            for (int e = 0; e < 4; e++) acc[k][e] += v[k][e];
          bool const more = j + 1 < cnt;
          uint32_t const next_id = j + 1 < kEmbChunk ? id1 : key_after;
          if (!more || next_id != id) {
            bool const tail_shared = !more && p1 < n && key_after == id;
            if (id != invalid_key) {
              if (shared_run || tail_shared) {
                // slot 2w: run shared with the previous walker (or both sides);
                // slot 2w+1: run shared with the next walker only
                int const slot = shared_run ? 2 * w : 2 * w + 1;
#pragma unroll
                for (int k = 0; k < CPL; k++) {
                  f32x4 pv = {acc[k][0], acc[k][1], acc[k][2], acc[k][3]};
                  *reinterpret_cast<f32x4 *>(emb_part + slot * PW + (k * LPR + wl) * 4) = pv;
                }
                if (wl == 0) {
                  part_id[slot] = id;
                  // 1: a border partial; 2 / 4: its run also extends before /
                  // beyond the workgroup's positions
                  part_valid[slot] = 1 | ((shared_run && p0 == block0) ? 2 : 0) |
                                     ((tail_shared && p1 == block1) ? 4 : 0);
                }
              } else {
#pragma unroll
                for (int k = 0; k < CPL; k++) {
                  int64_t const c = cbase + ((int64_t)k * LPR + wl) * 4;
                  if (c < dim) {
                    f32x4 upd = {o[k][0] + acc[k][0] * scale, o[k][1] + acc[k][1] * scale,
                                 o[k][2] + acc[k][2] * scale, o[k][3] + acc[k][3] * scale};
                    *reinterpret_cast<f32x4 *>(dW + (int64_t)id * dim + c) = upd;
                  }
                }
              }
            }
            shared_run = false;
#pragma unroll
            for (int k = 0; k < CPL; k++)
#pragma unroll
              for (int e = 0; e < 4; e++) acc[k][e] = 0.0f;
          }
        }
        // this slot is free now: position j + 2 goes into it
        prefetch(j + 2, id2, j + 3 < kEmbChunk ? id3 : key_after, l2, v, o);
        id0 = id1;
        id1 = id2;
        id2 = id3;
      };
#pragma unroll 1
      for (int j = 0; j < kEmbChunk; j += 2) {
        step(j, rows[0], old[0]);
        step(j + 1, rows[1], old[1]);
      }
    }
    __syncthreads();
    // merge the border partials in position order (first LPR threads, their column chunks)
    if (threadIdx.x < LPR) {
      float acc[CPL][4];
#pragma unroll
      for (int k = 0; k < CPL; k++)
#pragma unroll
        for (int e = 0; e < 4; e++) acc[k][e] = 0.0f;
      uint32_t cur_id = invalid_key;
      int flags = 0;
      for (int sidx = 0; sidx < 2 * WPB; sidx++) {
        int const v = part_valid[sidx];
        if (v == 0) continue;
        uint32_t const id = part_id[sidx];
        if (id != cur_id) {
          if (cur_id != invalid_key) add_row(cur_id, cbase, acc, (flags & 6) != 0);
          cur_id = id;
          flags = 0;
#pragma unroll
          for (int k = 0; k < CPL; k++)
#pragma unroll
            for (int e = 0; e < 4; e++) acc[k][e] = 0.0f;
        }
        flags |= v;
#pragma unroll
        for (int k = 0; k < CPL; k++) {
          f32x4 pv = *reinterpret_cast<f32x4 const *>(emb_part + sidx * PW + (k * LPR + wl) * 4);
#pragma unroll
          for (int e = 0; e < 4; e++) acc[k][e] += pv[e];
        }
      }
      if (cur_id != invalid_key) add_row(cur_id, cbase, acc, (flags & 6) != 0);
    }
    __syncthreads();
  }
}

// Scratch layout: keys A | keys B | lookups A | lookups B | digit table of the sort
struct EmbSortLayout {
  size_t keys_a, keys_b, vals_a, vals_b, table, total;
  RadixSortPlan plan;
};

static unsigned key_bits(int64_t num_entries) {
  unsigned b = 1;
  while (b < 32 && ((int64_t)1 << b) <= num_entries) b++;
  return b;
}

static bool emb_sort_layout(int64_t n, int64_t num_entries, EmbSortLayout &L) {
  if (n <= 0 || n >= (1ll << 31) || num_entries >= 0xffffffffll) return false;
  L.plan = radix_sort_plan(n, key_bits(num_entries));
  size_t const arr = ((size_t)n * 4 + 255) & ~(size_t)255;
  L.keys_a = 0;
  L.keys_b = arr;
  L.vals_a = 2 * arr;
  L.vals_b = 3 * arr;
  L.table = 4 * arr;
  L.total = 4 * arr + ((L.plan.table_bytes + 255) & ~(size_t)255);
  return true;
}

static int emb_grid(int64_t threads_needed) {
  int64_t b = ceil_div(threads_needed > 0 ? threads_needed : 1, kEmbThreads);
  int64_t const cap = (int64_t)kNumCU * 256;
  return (int)(b < cap ? b : cap);
}

template <typename IT, typename WT, typename OT>
static int emb_forward(hipStream_t st, void const *indices, void *output,
                       void const *weight, int64_t num_bags, int64_t bag,
                       int64_t dim, int64_t num_entries, float scale) {
  constexpr int V = emb_vec<WT, OT>();
  IT const *I = static_cast<IT const *>(indices);
  WT const *W = static_cast<WT const *>(weight);
  OT *O = static_cast<OT *>(output);
  if (dim % V == 0 && aligned16(weight) && aligned16(output)) {
    int nvec = (int)(dim / V);
    // 32-bit thread indices while index + one grid stride cannot wrap
    bool const fast = num_bags * nvec < ((int64_t)1 << 31) - (int64_t)kNumCU * 256 * kEmbThreads;
    FastDiv const by_nvec = fast ? make_fast_div((uint32_t)nvec) : FastDiv{};
#define FFK_EMB_FWD(BIG_, CHUNKED_)                                                                   \
  embedding_fwd_vec_kernel<IT, WT, OT, BIG_, CHUNKED_><<<emb_grid(num_bags * nvec), kEmbThreads, 0, st>>>( \
      I, O, W, num_bags, (int)bag, nvec, dim, num_entries, scale, by_nvec)
    if (bag >= 8) {
      if (fast) FFK_EMB_FWD(false, true);
      else FFK_EMB_FWD(true, true);
    } else {
      if (fast) FFK_EMB_FWD(false, false);
      else FFK_EMB_FWD(true, false);
    }
#undef FFK_EMB_FWD
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
                        int64_t num_entries, float scale, void *workspace,
                        size_t workspace_bytes, bool deterministic) {
  int64_t const lookups = num_bags * bag;
  EmbSortLayout L;
  bool const sorted = workspace != nullptr && dim % 4 == 0 &&
                      reinterpret_cast<uintptr_t>(dy) % 16 == 0 &&
                      reinterpret_cast<uintptr_t>(dw) % 16 == 0 &&
                      reinterpret_cast<uintptr_t>(workspace) % 256 == 0 &&
                      emb_sort_layout(lookups, num_entries, L) && L.total <= workspace_bytes;
  if (sorted) {
    uint8_t *ws = static_cast<uint8_t *>(workspace);
    uint32_t *keys_out = nullptr, *vals_out = nullptr;
    FFK_HIP(radix_sort_lookups<IT>(st, static_cast<IT const *>(indices), lookups, num_entries, L.plan,
                                   reinterpret_cast<uint32_t *>(ws + L.keys_a), reinterpret_cast<uint32_t *>(ws + L.keys_b),
                                   reinterpret_cast<uint32_t *>(ws + L.vals_a), reinterpret_cast<uint32_t *>(ws + L.vals_b),
                                   reinterpret_cast<uint32_t *>(ws + L.table), &keys_out, &vals_out));
    GT const *G = static_cast<GT const *>(dy);
    int64_t const walkers = ceil_div(lookups, kEmbChunk);
#define FFK_EMB_SORTED(LPR_, CPL_)                                             \
  do {                                                                         \
    if (deterministic) {                                                       \
      unsigned const blocks = (unsigned)ceil_div(walkers * LPR_, 256);         \
      embedding_bwd_sorted_kernel<GT, LPR_, CPL_, true><<<blocks, 256, 0, st>>>( \
          keys_out, vals_out, G, dw, lookups, (int)bag, dim, (uint32_t)num_entries, scale); \
    } else {                                                                   \
      unsigned const blocks = (unsigned)ceil_div(walkers * LPR_, kEmbBlockThreads); \
      auto kern = embedding_bwd_sorted_block_kernel<GT, LPR_, CPL_>;           \
      int const lds = 2 * (kEmbBlockThreads / LPR_) * LPR_ * 4 * CPL_ * (int)sizeof(float); \
      FFK_HIP(hipFuncSetAttribute(reinterpret_cast<void const *>(kern),        \
                                  hipFuncAttributeMaxDynamicSharedMemorySize, lds)); \
      kern<<<blocks, kEmbBlockThreads, lds, st>>>(                             \
          keys_out, vals_out, G, dw, lookups, (int)bag, dim, (uint32_t)num_entries, scale); \
    }                                                                          \
  } while (0)
    if (dim > 512) FFK_EMB_SORTED(64, 4);
    else if (dim > 256) FFK_EMB_SORTED(64, 2);
    else if (dim > 128) FFK_EMB_SORTED(64, 1);
    else if (dim > 64) FFK_EMB_SORTED(32, 1);
    else FFK_EMB_SORTED(16, 1);
#undef FFK_EMB_SORTED
    FFK_CHECK_LAUNCH();
    return FFK_OK;
  }
  if (deterministic) {
    return fail(FFK_ERR_WORKSPACE,
                "embedding_backward: deterministic mode needs the sort workspace "
                "(ffk_embedding_backward_workspace_bytes), 256-byte aligned, and dim %% 4 == 0");
  }
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
  if (weight_dtype == output_dtype && (weight_dtype == FFK_HALF || weight_dtype == FFK_DOUBLE) &&
      (index_dtype == FFK_INT32 || index_dtype == FFK_INT64)) {
    bool const avg = aggr == FFK_AGGR_AVG;
    int const grid = emb_grid(num_bags * dim);
#define FFK_EMB_TYPED(IT, T)                                                   \
  embedding_fwd_typed_kernel<IT, T><<<grid, kEmbThreads, 0, st>>>(             \
      static_cast<IT const *>(indices), static_cast<T *>(output), static_cast<T const *>(weight), num_bags, (int)bag, \
      dim, num_entries, avg)
    if (index_dtype == FFK_INT32 && weight_dtype == FFK_HALF) FFK_EMB_TYPED(int32_t, _Float16);
    else if (index_dtype == FFK_INT32) FFK_EMB_TYPED(int32_t, double);
    else if (weight_dtype == FFK_HALF) FFK_EMB_TYPED(int64_t, _Float16);
    else FFK_EMB_TYPED(int64_t, double);
#undef FFK_EMB_TYPED
    FFK_CHECK_LAUNCH();
    return FFK_OK;
  }
  return fail(FFK_ERR_UNSUPPORTED,
              "embedding_forward: dtypes (index %d, weight %d, output %d) not supported",
              index_dtype, weight_dtype, output_dtype);
}

extern "C" size_t ffk_embedding_backward_workspace_bytes(int64_t num_indices,
                                                         int64_t num_entries) {
  EmbSortLayout L;
  if (!emb_sort_layout(num_indices, num_entries, L)) return 0;
  return L.total;
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
  float scale = aggr == FFK_AGGR_AVG ? 1.0f / (float)bag : 1.0f;
  hipStream_t st = as_stream(stream);
#define FFK_EMB_BWD(IT, GT)                                                    \
  return emb_backward<IT, GT>(st, indices, output_grad, weight_grad, num_bags, bag, dim, num_entries, scale, \
                              workspace, workspace_bytes, deterministic != 0)
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

extern "C" int ffk_embedding_backward_typed(ffk_stream_t stream, int index_dtype, int dtype,
                                            void const *indices, void const *output_grad,
                                            void *weight_grad, int aggr, int64_t num_bags,
                                            int64_t bag, int64_t dim, int64_t num_entries) {
  if (dtype == FFK_FLOAT) {
    return ffk_embedding_backward(stream, index_dtype, FFK_FLOAT, indices, output_grad,
                                  static_cast<float *>(weight_grad), aggr, num_bags, bag, dim, num_entries, 0,
                                  nullptr, 0);
  }
  int rc = check_common("embedding_backward_typed", aggr, num_bags, bag, dim, num_entries);
  if (rc != FFK_OK) return rc;
  FFK_REQUIRE(dtype == FFK_HALF || dtype == FFK_DOUBLE,
              "embedding_backward_typed: dtype %d not supported (HALF, FLOAT or DOUBLE)", dtype);
  FFK_REQUIRE(index_dtype == FFK_INT32 || index_dtype == FFK_INT64,
              "embedding_backward_typed: index dtype %d not supported", index_dtype);
  if (num_bags == 0) return FFK_OK;
  FFK_REQUIRE(indices && output_grad && weight_grad, "embedding_backward_typed: NULL tensor");
  hipStream_t st = as_stream(stream);
  bool const avg = aggr == FFK_AGGR_AVG;
  int const grid = emb_grid(num_bags * dim);
#define FFK_EMB_TYPED(IT, T)                                                   \
  embedding_bwd_typed_kernel<IT, T><<<grid, kEmbThreads, 0, st>>>(             \
      static_cast<IT const *>(indices), static_cast<T const *>(output_grad), static_cast<T *>(weight_grad), num_bags, \
      (int)bag, dim, num_entries, avg)
  if (index_dtype == FFK_INT32 && dtype == FFK_HALF) FFK_EMB_TYPED(int32_t, _Float16);
  else if (index_dtype == FFK_INT32) FFK_EMB_TYPED(int32_t, double);
  else if (dtype == FFK_HALF) FFK_EMB_TYPED(int64_t, _Float16);
  else FFK_EMB_TYPED(int64_t, double);
#undef FFK_EMB_TYPED
  FFK_CHECK_LAUNCH();
  return FFK_OK;
}
