// The reference generates this header from softmax_per_device_state.dtg.toml; here the state struct
// is declared next to the entry points that use it.
#pragma once
#include "kernels/softmax_kernels.h"
