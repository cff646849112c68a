// DataType (reference: lib/op-attrs/include/op-attrs/datatype.dtg.toml:11-27;
// sizes lib/op-attrs/src/op-attrs/datatype.cc:8-24).  BF16 is appended so the
// reference's ordinals keep their values.
// data_type_enum_to_class / real_type_t / type_to_data_type_enum follow
// lib/op-attrs/include/op-attrs/datatype.h:12-66; the 16-bit types are plain
// storage (host code moves them, device code computes with them).
#pragma once
#include <cstddef>
#include <cstdint>
#include <stdexcept>
#include <type_traits>
namespace FlexFlow {
enum class DataType { BOOL, INT32, INT64, HALF, FLOAT, DOUBLE, BF16 };

struct half { uint16_t bits; };      // IEEE binary16 storage
struct bfloat16 { uint16_t bits; };  // upper half of an IEEE binary32

template <DataType>
struct data_type_enum_to_class;
template <> struct data_type_enum_to_class<DataType::FLOAT> { using type = float; };
template <> struct data_type_enum_to_class<DataType::DOUBLE> { using type = double; };
template <> struct data_type_enum_to_class<DataType::INT32> { using type = int32_t; };
template <> struct data_type_enum_to_class<DataType::INT64> { using type = int64_t; };
template <> struct data_type_enum_to_class<DataType::HALF> { using type = half; };
template <> struct data_type_enum_to_class<DataType::BOOL> { using type = bool; };
template <> struct data_type_enum_to_class<DataType::BF16> { using type = bfloat16; };

template <DataType DT>
using real_type_t = typename data_type_enum_to_class<DT>::type;

template <typename T>
struct type_to_data_type_enum;
template <> struct type_to_data_type_enum<double> : std::integral_constant<DataType, DataType::DOUBLE> {};
template <> struct type_to_data_type_enum<float> : std::integral_constant<DataType, DataType::FLOAT> {};
template <> struct type_to_data_type_enum<half> : std::integral_constant<DataType, DataType::HALF> {};
template <> struct type_to_data_type_enum<bfloat16> : std::integral_constant<DataType, DataType::BF16> {};
template <> struct type_to_data_type_enum<int32_t> : std::integral_constant<DataType, DataType::INT32> {};
template <> struct type_to_data_type_enum<int64_t> : std::integral_constant<DataType, DataType::INT64> {};
template <> struct type_to_data_type_enum<bool> : std::integral_constant<DataType, DataType::BOOL> {};
template <typename T>
inline constexpr DataType type_to_data_type_enum_v = type_to_data_type_enum<T>::value;

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
