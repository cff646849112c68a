// The reference generates this header from device_handle_t.dtg.toml; here the type is written by hand.
#pragma once
#include "kernels/device_handle_t.h"
