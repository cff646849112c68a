// Stable least-significant-digit radix sort of (row id, lookup number) pairs
// on the device, for the sorted embedding backward: rows that are looked up
// several times end up next to each other, in ascending lookup order.
//
// One pass sorts by 8 bits of the key and is three launches:
//   histogram  a workgroup counts the digits of its tile of 2048 keys into
//              table[digit][tile] and adds them to the digit totals of the pass;
//   scan       workgroup d turns row d of the table into exclusive prefix sums
//              on top of the totals of the digits below d: entry (d, t) becomes
//              the first output position of tile t's keys with digit d;
//   scatter    the workgroup re-reads its tile; each of its four waves owns a
//              quarter of it and walks that quarter 64 keys at a time in order,
//              ranking the keys of a step among their peers with the same digit
//              by ballots, so equal digits keep their input order (stable) and
//              the result does not depend on timing (no atomics decide a place).
// Up to kSortFusedTiles tiles (131 072 lookups) a pass is ONE launch: the scan
// moves into the scatter kernel (every workgroup adds up the counts of the
// tiles before its own and the totals of the digits below, straight from a
// table that is only a few tens of kilobytes), and the scatter counts the NEXT
// pass's digits of the keys it places, per destination tile, with integer
// atomics (a count does not depend on the order of the additions; the counts
// are gathered in LDS first, since under a skewed id distribution thousands of
// a workgroup's keys share one counter).  A sort of
// the token table's lookups is then 3 launches instead of 7.
// The first pass reads the caller's index tensor directly (int32 or int64,
// ids outside the table become the key `invalid_key`, which sorts behind every
// row) and numbers the lookups itself, so no pass exists only to build keys.
#pragma once
#include "ffk_common.h"

namespace ffk {

constexpr int kSortThreads = 256;
constexpr int kSortItems = 8;                              // keys per thread
constexpr int kSortTile = kSortThreads * kSortItems;       // keys per workgroup
constexpr int kSortRadix = 256;
constexpr int kSortWaveKeys = kSortTile / 4;               // keys per wave

template <typename IT, bool FIRST>
__device__ __forceinline__ uint32_t sort_key_at(IT const *idx, uint32_t const *keys_in, int64_t i,
                                                int64_t num_entries) {
  if constexpr (FIRST) {
    int64_t const r = (int64_t)idx[i];
    return (uint64_t)r < (uint64_t)num_entries ? (uint32_t)r : (uint32_t)num_entries;
  } else {
    return keys_in[i];
  }
}

template <typename IT, bool FIRST>
__global__ __launch_bounds__(kSortThreads) void radix_hist_kernel(IT const *__restrict__ idx,
                                                                  uint32_t const *__restrict__ keys_in,
                                                                  uint32_t *__restrict__ table,
                                                                  uint32_t *__restrict__ totals, int64_t n,
                                                                  int ntiles, int shift, int64_t num_entries) {
  __shared__ uint32_t cnt[kSortRadix];
  cnt[threadIdx.x] = 0;
  __syncthreads();
  int64_t const base = (int64_t)blockIdx.x * kSortTile;
#pragma unroll
  for (int k = 0; k < kSortItems; k++) {
    int64_t const i = base + k * kSortThreads + threadIdx.x;
    if (i < n) {
      uint32_t const key = sort_key_at<IT, FIRST>(idx, keys_in, i, num_entries);
      atomicAdd(&cnt[(key >> shift) & (kSortRadix - 1)], 1u);  // LDS; a count does not depend on order
    }
  }
  __syncthreads();
  uint32_t const c = cnt[threadIdx.x];
  table[(int64_t)threadIdx.x * ntiles + blockIdx.x] = c;
  if (c != 0) atomicAdd(&totals[threadIdx.x], c);  // integer sums: the order of the additions does not matter
}

__global__ __launch_bounds__(256) void radix_zero_kernel(uint32_t *p, int count) {
  int const i = blockIdx.x * 256 + threadIdx.x;
  if (i < count) p[i] = 0;
}

// Workgroup d: row d of the table (ntiles counts) becomes exclusive prefix sums
// that start at the number of keys whose digit is below d.
__global__ __launch_bounds__(kSortThreads) void radix_scan_kernel(uint32_t *table, uint32_t const *__restrict__ totals,
                                                                  int ntiles) {
  __shared__ uint32_t wsum[4];
  int const t = threadIdx.x, lane = t & 63, wave = t >> 6, d = blockIdx.x;
  auto block_sum = [&](uint32_t v) {  // every thread gets the total
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    __syncthreads();  // wsum may still be read from the previous use
    if (lane == 0) wsum[wave] = v;
    __syncthreads();
    return wsum[0] + wsum[1] + wsum[2] + wsum[3];
  };
  uint32_t carry = block_sum(t < d ? totals[t] : 0u);
  uint32_t *row = table + (int64_t)d * ntiles;
  for (int c0 = 0; c0 < ntiles; c0 += kSortThreads) {
    int const i = c0 + t;
    uint32_t const x = i < ntiles ? row[i] : 0u;
    uint32_t incl = x;  // inclusive scan inside the wave
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      uint32_t const up = __shfl_up(incl, off, 64);
      if (lane >= off) incl += up;
    }
    __syncthreads();
    if (lane == 63) wsum[wave] = incl;
    __syncthreads();
    uint32_t before = 0;
#pragma unroll
    for (int w = 0; w < 4; w++) before += w < wave ? wsum[w] : 0u;
    if (i < ntiles) row[i] = carry + before + incl - x;
    carry += wsum[0] + wsum[1] + wsum[2] + wsum[3];
  }
}

template <typename IT, bool FIRST>
__global__ __launch_bounds__(kSortThreads) void radix_scatter_kernel(
    IT const *__restrict__ idx, uint32_t const *__restrict__ keys_in, uint32_t const *__restrict__ vals_in,
    uint32_t *__restrict__ keys_out, uint32_t *__restrict__ vals_out, uint32_t const *__restrict__ table, int64_t n,
    int ntiles, int shift, int64_t num_entries) {
  __shared__ uint32_t wave_off[4][kSortRadix];  // per wave: digit counts, then the next free output position
  int const t = threadIdx.x, lane = t & 63, wave = t >> 6;
  for (int d = lane; d < kSortRadix; d += 64) wave_off[wave][d] = 0;
  // the zeroing above and the counting below touch this wave's row only, in program order
  int64_t const first = (int64_t)blockIdx.x * kSortTile + (int64_t)wave * kSortWaveKeys;
  constexpr int STEPS = kSortWaveKeys / 64;
  uint32_t key[STEPS], val[STEPS];
#pragma unroll
  for (int c = 0; c < STEPS; c++) {
    int64_t const i = first + c * 64 + lane;
    key[c] = 0;
    val[c] = 0;
    if (i < n) {
      key[c] = sort_key_at<IT, FIRST>(idx, keys_in, i, num_entries);
      val[c] = FIRST ? (uint32_t)i : vals_in[i];
      atomicAdd(&wave_off[wave][(key[c] >> shift) & (kSortRadix - 1)], 1u);
    }
  }
  __syncthreads();
  {
    // thread d: where each wave's keys with digit d start
    uint32_t run = table[(int64_t)t * ntiles + blockIdx.x];
#pragma unroll
    for (int w = 0; w < 4; w++) {
      uint32_t const c = wave_off[w][t];
      wave_off[w][t] = run;
      run += c;
    }
  }
  __syncthreads();
  uint64_t const below = ((uint64_t)1 << lane) - 1;
#pragma unroll
  for (int c = 0; c < STEPS; c++) {
    bool const valid = first + c * 64 + lane < n;
    uint32_t const digit = (key[c] >> shift) & (kSortRadix - 1);
    uint64_t peers = __ballot(valid);  // lanes of this step with this lane's digit
#pragma unroll
    for (int bit = 0; bit < 8; bit++) {
      uint64_t const m = __ballot((digit >> bit) & 1u);
      peers &= ((digit >> bit) & 1u) ? m : ~m;
    }
    if (valid) {
      uint32_t const start = wave_off[wave][digit];
      uint32_t const rank = (uint32_t)__popcll(peers & below);
      keys_out[start + rank] = key[c];
      vals_out[start + rank] = val[c];
      // LDS operations of a wave complete in program order: every peer has read `start`
      // before the first of them moves it on for the next step
      if (rank == 0) wave_off[wave][digit] = start + (uint32_t)__popcll(peers);
    }
  }
}

// ---------------------------------------------------------------------------
// The one-launch-per-pass form for few tiles.  Tables are [tile][digit], one per
// pass (pass p's is filled by the histogram kernel for p = 0 and by pass p-1's
// scatter otherwise; each kernel clears the table that the kernel after it adds
// into, so no launch exists only to clear).
// ---------------------------------------------------------------------------
constexpr int kSortFusedTiles = 48;  // a workgroup keeps its next-pass counts [tiles][256] in LDS

template <typename IT>
__global__ __launch_bounds__(kSortThreads) void radix_hist0_fused_kernel(IT const *__restrict__ idx,
                                                                        uint32_t *__restrict__ table0,
                                                                        uint32_t *__restrict__ table1, int64_t n,
                                                                        int64_t num_entries) {
  __shared__ uint32_t cnt[kSortRadix];
  cnt[threadIdx.x] = 0;
  __syncthreads();
  int64_t const base = (int64_t)blockIdx.x * kSortTile;
#pragma unroll
  for (int k = 0; k < kSortItems; k++) {
    int64_t const i = base + k * kSortThreads + threadIdx.x;
    if (i < n) {
      uint32_t const key = sort_key_at<IT, true>(idx, nullptr, i, num_entries);
      atomicAdd(&cnt[key & (kSortRadix - 1)], 1u);
    }
  }
  __syncthreads();
  table0[(int64_t)blockIdx.x * kSortRadix + threadIdx.x] = cnt[threadIdx.x];
  if (table1 != nullptr) table1[(int64_t)blockIdx.x * kSortRadix + threadIdx.x] = 0;
}

// table: this pass's counts; next: the next pass's table (nullptr on the last pass), added
// into here; after: the table of the pass after that (nullptr if none), cleared here.
template <typename IT, bool FIRST>
__global__ __launch_bounds__(kSortThreads) void radix_scatter_fused_kernel(
    IT const *__restrict__ idx, uint32_t const *__restrict__ keys_in, uint32_t const *__restrict__ vals_in,
    uint32_t *__restrict__ keys_out, uint32_t *__restrict__ vals_out, uint32_t const *__restrict__ table,
    uint32_t *__restrict__ next, uint32_t *__restrict__ after, int64_t n, int ntiles, int shift, int64_t num_entries) {
  __shared__ uint32_t wave_off[4][kSortRadix];
  __shared__ uint32_t wsum[4];
  __shared__ uint32_t next_cnt[kSortFusedTiles][kSortRadix];  // this workgroup's share of the next pass's table
  int const t = threadIdx.x, lane = t & 63, wave = t >> 6;
  for (int d = lane; d < kSortRadix; d += 64) wave_off[wave][d] = 0;
  if (next != nullptr) {
    for (int r = 0; r < ntiles; r++) next_cnt[r][t] = 0;
  }
  int64_t const first = (int64_t)blockIdx.x * kSortTile + (int64_t)wave * kSortWaveKeys;
  constexpr int STEPS = kSortWaveKeys / 64;
  uint32_t key[STEPS], val[STEPS];
#pragma unroll
  for (int c = 0; c < STEPS; c++) {
    int64_t const i = first + c * 64 + lane;
    key[c] = 0;
    val[c] = 0;
    if (i < n) {
      key[c] = sort_key_at<IT, FIRST>(idx, keys_in, i, num_entries);
      val[c] = FIRST ? (uint32_t)i : vals_in[i];
      atomicAdd(&wave_off[wave][(key[c] >> shift) & (kSortRadix - 1)], 1u);
    }
  }
  // thread d: the keys with digit d in the tiles before this one, and in all tiles
  uint32_t before_tiles = 0, all_tiles = 0;
  {
    int const tile = blockIdx.x;
    for (int t0 = 0; t0 < ntiles; t0 += 8) {
      uint32_t v[8];
#pragma unroll
      for (int u = 0; u < 8; u++) v[u] = t0 + u < ntiles ? table[(int64_t)(t0 + u) * kSortRadix + t] : 0u;
#pragma unroll
      for (int u = 0; u < 8; u++) {
        all_tiles += v[u];
        before_tiles += t0 + u < tile ? v[u] : 0u;
      }
    }
  }
  if (after != nullptr) after[(int64_t)blockIdx.x * kSortRadix + t] = 0;
  // exclusive scan of all_tiles over the digits: the keys with a smaller digit
  uint32_t incl = all_tiles;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    uint32_t const up = __shfl_up(incl, off, 64);
    if (lane >= off) incl += up;
  }
  if (lane == 63) wsum[wave] = incl;
  __syncthreads();  // also orders the wave_off counts above before their use below
  uint32_t smaller = incl - all_tiles;
#pragma unroll
  for (int w = 0; w < 4; w++) smaller += w < wave ? wsum[w] : 0u;
  {
    uint32_t run = smaller + before_tiles;
#pragma unroll
    for (int w = 0; w < 4; w++) {
      uint32_t const c = wave_off[w][t];
      wave_off[w][t] = run;
      run += c;
    }
  }
  __syncthreads();
  uint64_t const below = ((uint64_t)1 << lane) - 1;
#pragma unroll
  for (int c = 0; c < STEPS; c++) {
    bool const valid = first + c * 64 + lane < n;
    uint32_t const digit = (key[c] >> shift) & (kSortRadix - 1);
    uint64_t peers = __ballot(valid);
#pragma unroll
    for (int bit = 0; bit < 8; bit++) {
      uint64_t const m = __ballot((digit >> bit) & 1u);
      peers &= ((digit >> bit) & 1u) ? m : ~m;
    }
    if (valid) {
      uint32_t const start = wave_off[wave][digit];
      uint32_t const rank = (uint32_t)__popcll(peers & below);
      uint32_t const pos = start + rank;
      keys_out[pos] = key[c];
      vals_out[pos] = val[c];
      // the next pass's count of this key, in the tile it has just been placed in
      if (next != nullptr) atomicAdd(&next_cnt[pos / kSortTile][(key[c] >> (shift + 8)) & (kSortRadix - 1)], 1u);
      if (rank == 0) wave_off[wave][digit] = start + (uint32_t)__popcll(peers);
    }
  }
  if (next != nullptr) {
    __syncthreads();
    for (int r = 0; r < ntiles; r++) {
      uint32_t const c = next_cnt[r][t];
      if (c != 0) atomicAdd(&next[(int64_t)r * kSortRadix + t], c);
    }
  }
}

struct RadixSortPlan {
  int passes;
  int ntiles;
  bool fused;          // one launch per pass (few tiles)
  size_t table_bytes;  // fused: one [ntiles][256] table per pass; otherwise one [256][ntiles] table, then the digit totals [passes][256]
};

static inline RadixSortPlan radix_sort_plan(int64_t n, unsigned key_bits) {
  RadixSortPlan p;
  p.passes = (int)((key_bits + 7) / 8);
  p.ntiles = (int)ceil_div(n, kSortTile);
  p.fused = p.ntiles <= kSortFusedTiles;
  p.table_bytes = p.fused ? (size_t)kSortRadix * (size_t)p.ntiles * (size_t)p.passes * sizeof(uint32_t)
                          : (size_t)kSortRadix * ((size_t)p.ntiles + (size_t)p.passes) * sizeof(uint32_t);
  return p;
}

// Sorts the n lookups of `idx` by row id.  bufs: two key arrays and two value
// arrays of n entries each, and the table of plan.table_bytes.  On return
// *keys_sorted / *vals_sorted point at the arrays that hold the result.
template <typename IT>
static inline hipError_t radix_sort_lookups(hipStream_t st, IT const *idx, int64_t n, int64_t num_entries,
                                            RadixSortPlan const &plan, uint32_t *keys_a, uint32_t *keys_b,
                                            uint32_t *vals_a, uint32_t *vals_b, uint32_t *table,
                                            uint32_t **keys_sorted, uint32_t **vals_sorted) {
  uint32_t *kin = nullptr, *vin = nullptr, *kout = keys_a, *vout = vals_a;
  if (plan.fused) {
    unsigned const blocks = (unsigned)plan.ntiles;
    size_t const tsz = (size_t)kSortRadix * plan.ntiles;
    auto tab = [&](int pass) -> uint32_t * { return pass < plan.passes ? table + (size_t)pass * tsz : nullptr; };
    radix_hist0_fused_kernel<IT><<<blocks, kSortThreads, 0, st>>>(idx, tab(0), tab(1), n, num_entries);
    for (int pass = 0; pass < plan.passes; pass++) {
      int const shift = 8 * pass;
      if (pass == 0) {
        radix_scatter_fused_kernel<IT, true><<<blocks, kSortThreads, 0, st>>>(
            idx, nullptr, nullptr, kout, vout, tab(0), tab(1), tab(2), n, plan.ntiles, shift, num_entries);
      } else {
        radix_scatter_fused_kernel<IT, false><<<blocks, kSortThreads, 0, st>>>(
            idx, kin, vin, kout, vout, tab(pass), tab(pass + 1), tab(pass + 2), n, plan.ntiles, shift, num_entries);
      }
      hipError_t const e = hipGetLastError();
      if (e != hipSuccess) return e;
      kin = kout;
      vin = vout;
      kout = kin == keys_a ? keys_b : keys_a;
      vout = vin == vals_a ? vals_b : vals_a;
    }
    *keys_sorted = kin;
    *vals_sorted = vin;
    return hipSuccess;
  }
  uint32_t *const totals_all = table + (size_t)kSortRadix * plan.ntiles;
  radix_zero_kernel<<<plan.passes, 256, 0, st>>>(totals_all, plan.passes * kSortRadix);
  for (int pass = 0; pass < plan.passes; pass++) {
    int const shift = 8 * pass;
    unsigned const blocks = (unsigned)plan.ntiles;
    uint32_t *const totals = totals_all + pass * kSortRadix;
    if (pass == 0) {
      radix_hist_kernel<IT, true><<<blocks, kSortThreads, 0, st>>>(idx, nullptr, table, totals, n, plan.ntiles, shift, num_entries);
    } else {
      radix_hist_kernel<IT, false><<<blocks, kSortThreads, 0, st>>>(idx, kin, table, totals, n, plan.ntiles, shift, num_entries);
    }
    radix_scan_kernel<<<kSortRadix, kSortThreads, 0, st>>>(table, totals, plan.ntiles);
    if (pass == 0) {
      radix_scatter_kernel<IT, true><<<blocks, kSortThreads, 0, st>>>(idx, nullptr, nullptr, kout, vout, table, n,
                                                                     plan.ntiles, shift, num_entries);
    } else {
      radix_scatter_kernel<IT, false><<<blocks, kSortThreads, 0, st>>>(idx, kin, vin, kout, vout, table, n,
                                                                      plan.ntiles, shift, num_entries);
    }
    hipError_t const e = hipGetLastError();
    if (e != hipSuccess) return e;
    kin = kout;
    vin = vout;
    kout = kin == keys_a ? keys_b : keys_a;
    vout = vin == vals_a ? vals_b : vals_a;
  }
  *keys_sorted = kin;
  *vals_sorted = vin;
  return hipSuccess;
}

}  // namespace ffk
