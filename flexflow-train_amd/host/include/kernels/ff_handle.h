// PerDeviceFFHandle (reference: lib/kernels/include/kernels/ff_handle.h:12-24).
#pragma once
#include "kernels/device.h"
#include <cstddef>

namespace FlexFlow {

struct PerDeviceFFHandle {
  ffHandle_t dnn;        // null: no vendor library behind these kernels
  ffblasHandle_t blas;   // null
  void *workSpace;
  size_t workSpaceSize;
  bool allowTensorOpMathConversion;
  ffStream_t stream;     // one stream per handle (the reference creates one per call)
};

}  // namespace FlexFlow
