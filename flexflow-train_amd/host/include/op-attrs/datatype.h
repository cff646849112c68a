// DataType (reference: lib/op-attrs/include/op-attrs/datatype.dtg.toml:11-27;
// sizes lib/op-attrs/src/op-attrs/datatype.cc:8-24).  BF16 is appended so the
// reference's ordinals keep their values.
#pragma once
#include <cstddef>
#include <stdexcept>
namespace FlexFlow {
enum class DataType { BOOL, INT32, INT64, HALF, FLOAT, DOUBLE, BF16 };

inline size_t size_of_datatype(DataType dt) {
  switch (dt) {
    case DataType::BOOL: return 1;
    case DataType::INT32: return 4;
    case DataType::INT64: return 8;
    case DataType::HALF: return 2;
    case DataType::FLOAT: return 4;
    case DataType::DOUBLE: return 8;
    case DataType::BF16: return 2;
  }
  throw std::runtime_error("Unknown DataType");
}
}  // namespace FlexFlow
