// create_local_allocator_for_device_type (reference:
// lib/kernels/include/kernels/create_local_allocator_for_device_type.h).
#pragma once
#include "kernels/allocation.h"
