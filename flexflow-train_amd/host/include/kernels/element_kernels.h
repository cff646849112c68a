// Both element-wise operator families in one include.
#pragma once
#include "kernels/element_binary_kernels.h"
#include "kernels/element_unary_kernels.h"
