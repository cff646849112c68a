// ProfilingSettings (reference: lib/kernels/include/kernels/profiling_settings.dtg.toml;
// the reference generates the header, here the struct is written by hand).
#pragma once

namespace FlexFlow {

struct ProfilingSettings {
  int warmup_iters;
  int measure_iters;
};

}  // namespace FlexFlow
