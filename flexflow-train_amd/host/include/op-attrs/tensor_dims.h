// TensorDims helpers (reference: lib/op-attrs/include/op-attrs/tensor_dims.h).
#pragma once
#include "op-attrs/tensor_shape.h"
