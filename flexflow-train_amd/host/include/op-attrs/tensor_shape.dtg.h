// The reference generates this header from tensor_shape.dtg.toml.
#pragma once
#include "op-attrs/tensor_shape.h"
