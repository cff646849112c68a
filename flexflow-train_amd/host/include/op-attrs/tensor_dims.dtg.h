// The reference generates this header from tensor_dims.dtg.toml.
#pragma once
#include "op-attrs/tensor_shape.h"
