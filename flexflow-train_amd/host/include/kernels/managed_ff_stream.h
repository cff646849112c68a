#pragma once
#include "kernels/device.h"

namespace FlexFlow {

// RAII stream (reference: lib/kernels/include/kernels/managed_ff_stream.h)
struct ManagedFFStream {
  ManagedFFStream();
  ManagedFFStream(ManagedFFStream const &) = delete;
  ManagedFFStream &operator=(ManagedFFStream const &) = delete;
  ManagedFFStream(ManagedFFStream &&other) noexcept;
  ~ManagedFFStream();
  ffStream_t const &raw_stream() const { return stream; }
 private:
  ffStream_t stream;
};

}  // namespace FlexFlow
