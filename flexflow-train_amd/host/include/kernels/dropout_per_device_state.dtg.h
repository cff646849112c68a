// The reference generates this header from dropout_per_device_state.dtg.toml; here the state struct
// is declared next to the entry points that use it.
#pragma once
#include "kernels/dropout_kernels.h"
