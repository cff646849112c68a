// The reference generates this header from datatype.dtg.toml.
#pragma once
#include "op-attrs/datatype.h"
