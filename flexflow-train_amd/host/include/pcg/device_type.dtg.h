// The reference generates this header from device_type.dtg.toml.
#pragma once
#include "pcg/device_type.h"
