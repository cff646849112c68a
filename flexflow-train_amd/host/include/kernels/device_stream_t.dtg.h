// The reference generates this header from device_stream_t.dtg.toml; here the type is written by hand.
#pragma once
#include "kernels/device_stream_t.h"
