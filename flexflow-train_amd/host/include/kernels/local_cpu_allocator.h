// LocalCPUAllocator (reference: lib/kernels/include/kernels/local_cpu_allocator.h;
// body lib/kernels/src/kernels/local_cpu_allocator.cc).
#pragma once
#include "kernels/allocation.h"
