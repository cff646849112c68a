// LocalCudaAllocator (reference: lib/kernels/include/kernels/local_cuda_allocator.h).
// The device allocator keeps the reference's name so callers compile unchanged.
#pragma once
#include "kernels/allocation.h"
