// Runtime shim of the C ABI: device memory, copies, streams and events.
// Host C++ above this library never includes a HIP header; these calls are
// what it uses instead of cudaMalloc/cudaMemcpy/cudaStreamCreate/cudaEvent*
// (reference: lib/kernels/src/kernels/local_cuda_allocator.cc,
// lib/kernels/src/kernels/accessor.cc:45-74,
// lib/kernels/include/kernels/profiling.h:78-106).
#include "ffk_common.h"
#include <atomic>
#include <stdarg.h>
#include <stdlib.h>
#include <string.h>

namespace ffk {

static thread_local char g_err[1024] = "";

void set_error(char const *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

int fail(int code, char const *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

// Process-wide switches: changed by ffk_set_option only (nothing in the
// library reads the environment), all 0 = the dispatch's own choices.
static std::atomic<int> g_option[FFK_OPTION_COUNT] = {{0}, {0}, {0}};
int option(int which) { return g_option[which].load(std::memory_order_relaxed); }

// Zero fill as a kernel (not hipMemsetAsync) so that callers may capture the
// call into a HIP graph.
__global__ void fill_zero_kernel(u32x4 *p16, size_t n16, uint8_t *tail,
                                 size_t ntail) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  size_t stride = (size_t)gridDim.x * blockDim.x;
  u32x4 z = {0u, 0u, 0u, 0u};
  for (size_t j = i; j < n16; j += stride) {
    p16[j] = z;
  }
  if (i < ntail) {
    tail[i] = 0;
  }
}

}  // namespace ffk

using namespace ffk;

extern "C" {

char const *ffk_last_error(void) { return g_err; }

int ffk_set_option(int which, int value) {
  FFK_REQUIRE(which >= 0 && which < FFK_OPTION_COUNT, "ffk_set_option: no option %d", which);
  g_option[which].store(value, std::memory_order_relaxed);
  return FFK_OK;
}

int ffk_get_option(int which, int *value) {
  FFK_REQUIRE(which >= 0 && which < FFK_OPTION_COUNT && value != nullptr, "ffk_get_option: no option %d", which);
  *value = option(which);
  return FFK_OK;
}

int ffk_device_count(int *count) {
  FFK_REQUIRE(count != nullptr, "ffk_device_count: count is NULL");
  FFK_HIP(hipGetDeviceCount(count));
  return FFK_OK;
}

int ffk_set_device(int device) {
  FFK_HIP(hipSetDevice(device));
  return FFK_OK;
}

int ffk_malloc(void **ptr, size_t bytes) {
  FFK_REQUIRE(ptr != nullptr, "ffk_malloc: ptr is NULL");
  *ptr = nullptr;
  if (bytes == 0) {
    return FFK_OK;
  }
  FFK_HIP(hipMalloc(ptr, bytes));
  return FFK_OK;
}

int ffk_free(void *ptr) {
  if (ptr != nullptr) {
    FFK_HIP(hipFree(ptr));
  }
  return FFK_OK;
}

int ffk_host_malloc(void **ptr, size_t bytes) {
  FFK_REQUIRE(ptr != nullptr, "ffk_host_malloc: ptr is NULL");
  FFK_HIP(hipHostMalloc(ptr, bytes, hipHostMallocDefault));
  return FFK_OK;
}

int ffk_host_free(void *ptr) {
  if (ptr != nullptr) {
    FFK_HIP(hipHostFree(ptr));
  }
  return FFK_OK;
}

int ffk_memcpy(void *dst, void const *src, size_t bytes, int kind,
               ffk_stream_t stream) {
  if (bytes == 0) {
    return FFK_OK;
  }
  FFK_REQUIRE(dst != nullptr && src != nullptr, "ffk_memcpy: NULL pointer");
  hipMemcpyKind k;
  switch (kind) {
    case FFK_H2D: k = hipMemcpyHostToDevice; break;
    case FFK_D2H: k = hipMemcpyDeviceToHost; break;
    case FFK_D2D: k = hipMemcpyDeviceToDevice; break;
    default: return fail(FFK_ERR_INVALID, "ffk_memcpy: bad kind %d", kind);
  }
  if (stream == nullptr) {
    FFK_HIP(hipMemcpy(dst, src, bytes, k));
  } else {
    FFK_HIP(hipMemcpyAsync(dst, src, bytes, k, as_stream(stream)));
  }
  return FFK_OK;
}

int ffk_fill_zero(void *ptr, size_t bytes, ffk_stream_t stream) {
  if (bytes == 0) {
    return FFK_OK;
  }
  FFK_REQUIRE(ptr != nullptr, "ffk_fill_zero: NULL pointer");
  uint8_t *p = static_cast<uint8_t *>(ptr);
  // Bytes before the first 16-byte boundary are cleared as part of the tail.
  size_t head = (16 - (reinterpret_cast<uintptr_t>(p) & 15u)) & 15u;
  if (head > bytes) {
    head = bytes;
  }
  if (head > 0) {
    fill_zero_kernel<<<1, 64, 0, as_stream(stream)>>>(nullptr, 0, p, head);
    FFK_CHECK_LAUNCH();
    p += head;
    bytes -= head;
  }
  size_t n16 = bytes / 16;
  size_t ntail = bytes % 16;
  if (n16 == 0 && ntail == 0) {
    return FFK_OK;
  }
  int64_t blocks = ceil_div((int64_t)(n16 > 0 ? n16 : 1), 256);
  if (blocks > kNumCU * 16) {
    blocks = kNumCU * 16;
  }
  fill_zero_kernel<<<(int)blocks, 256, 0, as_stream(stream)>>>(
      reinterpret_cast<u32x4 *>(p), n16, p + n16 * 16, ntail);
  FFK_CHECK_LAUNCH();
  return FFK_OK;
}

int ffk_stream_create(ffk_stream_t *stream) {
  FFK_REQUIRE(stream != nullptr, "ffk_stream_create: stream is NULL");
  hipStream_t s;
  FFK_HIP(hipStreamCreate(&s));  // default priority only
  *stream = reinterpret_cast<ffk_stream_t>(s);
  return FFK_OK;
}

int ffk_stream_destroy(ffk_stream_t stream) {
  if (stream != nullptr) {
    FFK_HIP(hipStreamDestroy(as_stream(stream)));
  }
  return FFK_OK;
}

int ffk_stream_synchronize(ffk_stream_t stream) {
  FFK_HIP(hipStreamSynchronize(as_stream(stream)));
  return FFK_OK;
}

int ffk_event_create(ffk_event_t *ev) {
  FFK_REQUIRE(ev != nullptr, "ffk_event_create: ev is NULL");
  hipEvent_t e;
  FFK_HIP(hipEventCreate(&e));
  *ev = reinterpret_cast<ffk_event_t>(e);
  return FFK_OK;
}

int ffk_event_destroy(ffk_event_t ev) {
  if (ev != nullptr) {
    FFK_HIP(hipEventDestroy(reinterpret_cast<hipEvent_t>(ev)));
  }
  return FFK_OK;
}

int ffk_event_record(ffk_event_t ev, ffk_stream_t stream) {
  FFK_HIP(hipEventRecord(reinterpret_cast<hipEvent_t>(ev), as_stream(stream)));
  return FFK_OK;
}

int ffk_event_synchronize(ffk_event_t ev) {
  FFK_HIP(hipEventSynchronize(reinterpret_cast<hipEvent_t>(ev)));
  return FFK_OK;
}

int ffk_event_elapsed_ms(ffk_event_t start, ffk_event_t stop, float *ms) {
  FFK_REQUIRE(ms != nullptr, "ffk_event_elapsed_ms: ms is NULL");
  FFK_HIP(hipEventElapsedTime(ms, reinterpret_cast<hipEvent_t>(start),
                              reinterpret_cast<hipEvent_t>(stop)));
  return FFK_OK;
}

}  // extern "C"
