// Accessor copies through an allocator (reference:
// lib/kernels/include/kernels/copy_tensor_accessor.h:9-25).
#pragma once
#include "kernels/allocation.h"
