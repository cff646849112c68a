// Concat forward/backward for gfx950 (reference: lib/kernels/src/cuda/ops/
// concat_kernels.cu:22-97, which launches copy_with_stride / add_with_stride
// once per input).  The output is viewed as [num_blocks, sum_i blk_i] and input
// i as [num_blocks, blk_i] (blk = product of the dims from the axis on).  Here
// one launch moves all inputs: a lane owns a fixed column range of the
// concatenated row, finds the input it falls into once (binary search over the
// prefix offsets, held in LDS), and then walks the rows.  Forward and the
// overwriting backward are byte moves (any data type, 16 bytes per lane when
// every blk_i and pointer allows); the accumulating backward adds in fp32.
#include "ffk_common.h"

namespace ffk {

constexpr int kConcatThreads = 256;
constexpr int kConcatMaxParts = 64;

struct ConcatArgs {
  char *part[kConcatMaxParts];
  int64_t offset[kConcatMaxParts + 1];  // byte offset of each part inside a concatenated row
  int parts;
  int cols_per_wg;      // units of a row one workgroup covers (<= kConcatThreads)
  int64_t units_per_row;  // units of the concatenated row this launch covers
  int64_t cat_row_bytes;  // bytes between consecutive concatenated rows
  int64_t num_blocks;
};

// gather: concatenated row <- parts; scatter: parts <- concatenated row; "Add" adds to the destination
enum ConcatMode { kGather = 0, kScatter = 1, kScatterAddF32 = 2, kScatterAddBf16 = 3, kGatherAddF32 = 4, kGatherAddBf16 = 5 };

// U: the unit a lane moves (uint8/16/32/64 or 16 bytes)
template <typename U, int MODE>
__global__ __launch_bounds__(kConcatThreads) void concat_kernel(char *cat, ConcatArgs a) {
  __shared__ int64_t offset[kConcatMaxParts + 1];
  __shared__ char *part[kConcatMaxParts];
  for (int i = threadIdx.x; i <= a.parts; i += kConcatThreads) {
    offset[i] = a.offset[i];
    if (i < a.parts) part[i] = a.part[i];
  }
  __syncthreads();
  int const rows_per_wg = kConcatThreads / a.cols_per_wg;
  int const r_local = threadIdx.x / a.cols_per_wg;
  int64_t const c = (int64_t)blockIdx.x * a.cols_per_wg + (threadIdx.x - r_local * a.cols_per_wg);
  if (c >= a.units_per_row || r_local >= rows_per_wg) return;
  int64_t const byte = c * (int64_t)sizeof(U);
  int lo = 0, hi = a.parts;  // offset[lo] <= byte < offset[hi]
  while (hi - lo > 1) {
    int const mid = (lo + hi) >> 1;
    if (offset[mid] <= byte) lo = mid;
    else hi = mid;
  }
  int64_t const part_row = offset[lo + 1] - offset[lo];
  int64_t const cat_row = a.cat_row_bytes;
  char *const p0 = part[lo] + (byte - offset[lo]);
  char *const c0 = cat + byte;
  int64_t const step = (int64_t)gridDim.y * rows_per_wg;
  for (int64_t row = (int64_t)blockIdx.y * rows_per_wg + r_local; row < a.num_blocks; row += step) {
    U *const pp = reinterpret_cast<U *>(p0 + row * part_row);
    U *const cp = reinterpret_cast<U *>(c0 + row * cat_row);
    if (MODE == kGather) {
      *cp = *pp;
    } else if (MODE == kScatter) {
      *pp = *cp;
    } else {
      // adding: src -> dst depends on the direction
      constexpr bool kToParts = MODE == kScatterAddF32 || MODE == kScatterAddBf16;
      U *const dst = kToParts ? pp : cp;
      U const *const src = kToParts ? cp : pp;
      if constexpr (MODE == kScatterAddF32 || MODE == kGatherAddF32) {
        // U is f32x4 or float
        *dst = *dst + *src;
      } else if constexpr (sizeof(U) == 16) {
        // 8 bf16: add in fp32, round once
        u32x4 const g = *reinterpret_cast<u32x4 const *>(src);
        u32x4 o = *reinterpret_cast<u32x4 *>(dst);
#pragma unroll
        for (int i = 0; i < 4; i++) {
          float const l = __uint_as_float(o[i] << 16) + __uint_as_float(g[i] << 16);
          float const h = __uint_as_float(o[i] & 0xffff0000u) + __uint_as_float(g[i] & 0xffff0000u);
          o[i] = pack_bf16x2(l, h);
        }
        *reinterpret_cast<u32x4 *>(dst) = o;
      } else {
        uint16_t const g = *reinterpret_cast<uint16_t const *>(src);
        uint16_t const o = *reinterpret_cast<uint16_t *>(dst);
        *reinterpret_cast<uint16_t *>(dst) = (uint16_t)f32_to_bf16_bits(bf16_bits_to_f32(o) + bf16_bits_to_f32(g));
      }
    }
  }
}

template <typename U, int MODE>
static hipError_t concat_launch(hipStream_t st, char *cat, ConcatArgs &a, int64_t window_bytes) {
  a.units_per_row = window_bytes / (int64_t)sizeof(U);
  a.cols_per_wg = (int)(a.units_per_row < kConcatThreads ? a.units_per_row : kConcatThreads);
  int const rows_per_wg = kConcatThreads / a.cols_per_wg;
  int64_t const gx = ceil_div(a.units_per_row, a.cols_per_wg);
  int64_t gy = ceil_div(a.num_blocks, rows_per_wg);
  // enough workgroups to fill the chip, rows beyond that are walked by the loop
  int64_t const want = (int64_t)kNumCU * 16;
  int64_t const cap = gx >= want ? 1 : ceil_div(want, gx);
  if (gy > cap) gy = cap;
  if (gy > 65535) gy = 65535;
  concat_kernel<U, MODE><<<dim3((unsigned)gx, (unsigned)gy), kConcatThreads, 0, st>>>(cat, a);
  return hipGetLastError();
}

static int elem_bytes(int dtype) {
  switch (dtype) {
    case FFK_BOOL: return 1;
    case FFK_HALF: case FFK_BF16: return 2;
    case FFK_INT32: case FFK_FLOAT: return 4;
    case FFK_INT64: case FFK_DOUBLE: return 8;
    default: return 0;
  }
}

// mode: 0 row <- parts, 1 parts <- row, 2 parts += row, 3 row += parts
static int concat_any(char const *who, ffk_stream_t stream, int dtype, void *cat, void *const *parts,
                      int64_t const *part_blk_elems, int num_parts, int64_t num_blocks, int mode) {
  int const eb = elem_bytes(dtype);
  FFK_REQUIRE(eb != 0, "%s: data type %d not supported", who, dtype);
  FFK_REQUIRE(num_parts >= 1 && num_blocks >= 0, "%s: bad sizes", who);
  FFK_REQUIRE(parts != nullptr && part_blk_elems != nullptr, "%s: NULL argument", who);
  FFK_REQUIRE(mode < 2 || dtype == FFK_FLOAT || dtype == FFK_BF16,
              "%s: accumulating backward supports float and bf16 (got data type %d)", who, dtype);
  hipStream_t st = as_stream(stream);
  int64_t row_bytes = 0;
  for (int i = 0; i < num_parts; i++) {
    FFK_REQUIRE(part_blk_elems[i] >= 0, "%s: negative block size", who);
    row_bytes += part_blk_elems[i] * eb;
  }
  if (num_blocks == 0 || row_bytes == 0) return FFK_OK;
  FFK_REQUIRE(cat != nullptr, "%s: NULL tensor", who);
  // parts are moved in groups of at most kConcatMaxParts; each group is a window of the row
  int64_t window_start = 0;
  for (int first = 0; first < num_parts; first += kConcatMaxParts) {
    int const n = num_parts - first < kConcatMaxParts ? num_parts - first : kConcatMaxParts;
    ConcatArgs a;
    a.parts = 0;
    a.num_blocks = num_blocks;
    a.cat_row_bytes = row_bytes;
    int64_t off = 0;
    bool wide = (reinterpret_cast<uintptr_t>(cat) + window_start) % 16 == 0 && row_bytes % 16 == 0;
    for (int i = 0; i < n; i++) {
      int64_t const bytes = part_blk_elems[first + i] * eb;
      if (bytes == 0) continue;  // empty parts take no room in the row
      FFK_REQUIRE(parts[first + i] != nullptr, "%s: NULL tensor", who);
      a.part[a.parts] = static_cast<char *>(parts[first + i]);
      a.offset[a.parts] = off;
      wide = wide && bytes % 16 == 0 && reinterpret_cast<uintptr_t>(parts[first + i]) % 16 == 0;
      off += bytes;
      a.parts++;
    }
    a.offset[a.parts] = off;
    if (a.parts > 0) {
      char *const base = static_cast<char *>(cat) + window_start;
      hipError_t e;
      if (mode == 0) {
        if (wide) e = concat_launch<u32x4, kGather>(st, base, a, off);
        else if (eb == 1) e = concat_launch<uint8_t, kGather>(st, base, a, off);
        else if (eb == 2) e = concat_launch<uint16_t, kGather>(st, base, a, off);
        else if (eb == 4) e = concat_launch<uint32_t, kGather>(st, base, a, off);
        else e = concat_launch<uint64_t, kGather>(st, base, a, off);
      } else if (mode == 1) {
        if (wide) e = concat_launch<u32x4, kScatter>(st, base, a, off);
        else if (eb == 1) e = concat_launch<uint8_t, kScatter>(st, base, a, off);
        else if (eb == 2) e = concat_launch<uint16_t, kScatter>(st, base, a, off);
        else if (eb == 4) e = concat_launch<uint32_t, kScatter>(st, base, a, off);
        else e = concat_launch<uint64_t, kScatter>(st, base, a, off);
      } else if (mode == 2 && dtype == FFK_FLOAT) {
        if (wide) e = concat_launch<f32x4, kScatterAddF32>(st, base, a, off);
        else e = concat_launch<float, kScatterAddF32>(st, base, a, off);
      } else if (mode == 2) {
        if (wide) e = concat_launch<u32x4, kScatterAddBf16>(st, base, a, off);
        else e = concat_launch<uint16_t, kScatterAddBf16>(st, base, a, off);
      } else if (dtype == FFK_FLOAT) {
        if (wide) e = concat_launch<f32x4, kGatherAddF32>(st, base, a, off);
        else e = concat_launch<float, kGatherAddF32>(st, base, a, off);
      } else {
        if (wide) e = concat_launch<u32x4, kGatherAddBf16>(st, base, a, off);
        else e = concat_launch<uint16_t, kGatherAddBf16>(st, base, a, off);
      }
      FFK_HIP(e);
    }
    window_start += off;
  }
  return FFK_OK;
}

}  // namespace ffk

using namespace ffk;

extern "C" int ffk_concat_forward(ffk_stream_t stream, int dtype, void *output, void const *const *inputs,
                                  int64_t const *input_blk_elems, int num_inputs, int64_t num_blocks) {
  return concat_any("concat_forward", stream, dtype, output, const_cast<void *const *>(reinterpret_cast<void const *const *>(inputs)),
                    input_blk_elems, num_inputs, num_blocks, 0);
}

extern "C" int ffk_concat_backward(ffk_stream_t stream, int dtype, void const *output_grad, void *const *input_grads,
                                   int64_t const *input_blk_elems, int num_inputs, int64_t num_blocks,
                                   int accumulate) {
  return concat_any("concat_backward", stream, dtype, const_cast<void *>(output_grad), input_grads, input_blk_elems,
                    num_inputs, num_blocks, accumulate ? 2 : 1);
}

// Split is Concat read the other way (reference: lib/kernels/src/cuda/ops/split_kernels.cu).
extern "C" int ffk_split_forward(ffk_stream_t stream, int dtype, void *const *outputs, void const *input,
                                 int64_t const *output_blk_elems, int num_outputs, int64_t num_blocks) {
  return concat_any("split_forward", stream, dtype, const_cast<void *>(input), outputs, output_blk_elems, num_outputs,
                    num_blocks, 1);
}

extern "C" int ffk_split_backward(ffk_stream_t stream, int dtype, void *input_grad, void const *const *output_grads,
                                  int64_t const *output_blk_elems, int num_outputs, int64_t num_blocks,
                                  int accumulate) {
  return concat_any("split_backward", stream, dtype, input_grad,
                    const_cast<void *const *>(reinterpret_cast<void const *const *>(output_grads)), output_blk_elems,
                    num_outputs, num_blocks, accumulate ? 3 : 0);
}
