// Opaque device handles for host code (reference: lib/kernels/include/kernels/
// device.h:4-82 typedefs cudaStream_t etc. from the CUDA headers; here no
// device header is included above the C ABI).
#pragma once
#include <stdexcept>
#include <string>

namespace FlexFlow {
using ffStream_t = void *;
using ffEvent_t = void *;
using ffHandle_t = void *;      // was cudnnHandle_t: unused, kept null
using ffblasHandle_t = void *;  // was cublasHandle_t: unused, kept null
using ffTensorDescriptor_t = void *;
using ffActivationDescriptor_t = void *;

// Device failures are fatal in the reference (FatalError -> abort,
// device.h:88-108); here they surface as this exception with the C ABI's text.
struct FatalError : std::runtime_error {
  using std::runtime_error::runtime_error;
};
void check_ffk(int status, char const *what);
}  // namespace FlexFlow
