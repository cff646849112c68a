// DeviceType (reference: lib/pcg/include/pcg/device_type.dtg.toml).
#pragma once
namespace FlexFlow {
enum class DeviceType { GPU, CPU };
}
