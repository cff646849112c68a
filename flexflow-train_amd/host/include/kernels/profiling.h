// profiling_wrapper (reference: lib/kernels/include/kernels/profiling.h:14-106):
// times f(stream, args...) with device events.  With measure_iters <= 0 the
// reference's settings overload returns nullopt WITHOUT calling f (:36-38);
// here f is called once, untimed, so a training loop given {0, 0} still runs.
#pragma once
#include "kernels/device_stream_t.h"
#include "kernels/profiling_settings.dtg.h"
#include <optional>
#include <utility>

extern "C" {
int ffk_event_create(void **ev);
int ffk_event_destroy(void *ev);
int ffk_event_record(void *ev, void *stream);
int ffk_event_synchronize(void *ev);
int ffk_event_elapsed_ms(void *start, void *stop, float *ms);
}

namespace FlexFlow {

struct milliseconds_t {
  float value;
};

template <typename F, typename... Ts>
milliseconds_t gpu_profiling_wrapper(F const &f, ProfilingSettings const &settings, Ts &&...ts) {
  device_stream_t stream = get_gpu_device_stream();
  ffEvent_t t_start = nullptr, t_end = nullptr;
  check_ffk(ffk_event_create(&t_start), "ffEventCreate");
  check_ffk(ffk_event_create(&t_end), "ffEventCreate");
  for (int i = 0; i < settings.warmup_iters + settings.measure_iters; i++) {
    if (i == settings.warmup_iters) {
      check_ffk(ffk_event_record(t_start, stream.require_gpu()), "ffEventRecord");
    }
    f(stream, std::forward<Ts>(ts)...);
  }
  float elapsed = 0;
  check_ffk(ffk_event_record(t_end, stream.require_gpu()), "ffEventRecord");
  check_ffk(ffk_event_synchronize(t_end), "ffEventSynchronize");
  check_ffk(ffk_event_elapsed_ms(t_start, t_end, &elapsed), "ffEventElapsedTime");
  ffk_event_destroy(t_start);
  ffk_event_destroy(t_end);
  return milliseconds_t{elapsed / settings.measure_iters};
}

template <typename F, typename... Ts>
std::optional<milliseconds_t> profiling_wrapper(F const &f, ProfilingSettings const &settings,
                                                DeviceType device_type, Ts &&...ts) {
  if (settings.measure_iters <= 0) {
    f(get_stream_for_device_type(device_type), std::forward<Ts>(ts)...);
    return std::nullopt;
  }
  if (device_type != DeviceType::GPU) {
    throw std::runtime_error("profiling_wrapper: the CPU device type is not executed by this library");
  }
  return gpu_profiling_wrapper(f, settings, std::forward<Ts>(ts)...);
}

template <typename F, typename... Ts>
std::optional<milliseconds_t> profiling_wrapper(F const &f, bool enable_profiling,
                                                DeviceType device_type, Ts &&...ts) {
  if (enable_profiling) {
    return profiling_wrapper(f, ProfilingSettings{0, 1}, device_type, std::forward<Ts>(ts)...);
  }
  f(get_stream_for_device_type(device_type), std::forward<Ts>(ts)...);
  return std::nullopt;
}

}  // namespace FlexFlow
