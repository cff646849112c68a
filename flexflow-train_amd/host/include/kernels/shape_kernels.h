// Transpose, Reshape, Split and Gather in one include.
#pragma once
#include "kernels/gather_kernels.h"
#include "kernels/reshape_kernels.h"
#include "kernels/split_kernels.h"
#include "kernels/transpose_kernels.h"
