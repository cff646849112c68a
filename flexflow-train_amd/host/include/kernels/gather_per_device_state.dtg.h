// The reference generates this header from gather_per_device_state.dtg.toml; here the state struct
// is declared next to the entry points that use it.
#pragma once
#include "kernels/gather_kernels.h"
