// The reference generates this header from element_unary_per_device_state.dtg.toml; here the state struct
// is declared next to the entry points that use it.
#pragma once
#include "kernels/element_unary_kernels.h"
