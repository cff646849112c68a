// GenericTensorAccessorR/W (reference: lib/kernels/include/kernels/accessor.h:
// 22-140; offsets lib/kernels/src/kernels/accessor.cc:15-33; copies :45-74).
#pragma once
#include "op-attrs/tensor_shape.h"
#include "pcg/device_type.h"
#include <optional>
#include <stdexcept>
#include <vector>

namespace FlexFlow {

using TensorDimsCoord = std::vector<int64_t>;

// Row-major offset with the reference's checks: rank must match, every index
// in bounds; throws otherwise.
int64_t calculate_accessor_offset(TensorDimsCoord const &coord, TensorDims const &dims);

struct GenericTensorAccessorR {
  TensorShape shape;
  void const *ptr;
  DeviceType device_type;

  float const *get_float_ptr() const { return typed<float>(DataType::FLOAT); }
  int32_t const *get_int32_ptr() const { return typed<int32_t>(DataType::INT32); }
  int64_t const *get_int64_ptr() const { return typed<int64_t>(DataType::INT64); }

  // Element access on a CPU-resident accessor (asserts residency and dtype).
  template <typename T>
  T const &at(TensorDimsCoord const &coord) const {
    if (device_type != DeviceType::CPU) throw std::runtime_error("at() requires a CPU accessor");
    if (sizeof(T) != size_of_datatype(shape.data_type)) throw std::runtime_error("at(): dtype mismatch");
    return static_cast<T const *>(ptr)[calculate_accessor_offset(coord, shape.dims)];
  }

 private:
  template <typename T>
  T const *typed(DataType want) const {
    if (shape.data_type != want) throw std::runtime_error("accessor: invalid data type");
    return static_cast<T const *>(ptr);
  }
};

struct GenericTensorAccessorW {
  TensorShape shape;
  void *ptr;
  DeviceType device_type;

  operator GenericTensorAccessorR() const { return GenericTensorAccessorR{shape, ptr, device_type}; }
  float *get_float_ptr() const {
    if (shape.data_type != DataType::FLOAT) throw std::runtime_error("accessor: invalid data type");
    return static_cast<float *>(ptr);
  }
  template <typename T>
  T &at(TensorDimsCoord const &coord) const {
    if (device_type != DeviceType::CPU) throw std::runtime_error("at() requires a CPU accessor");
    if (sizeof(T) != size_of_datatype(shape.data_type)) throw std::runtime_error("at(): dtype mismatch");
    return static_cast<T *>(ptr)[calculate_accessor_offset(coord, shape.dims)];
  }
};

GenericTensorAccessorR read_only_accessor_from_write_accessor(GenericTensorAccessorW const &);
TensorShape get_tensor_shape_for_accessor_r(GenericTensorAccessorR const &);
TensorShape get_tensor_shape_for_accessor_w(GenericTensorAccessorW const &);

// dst <- src for any pairing of CPU/GPU residency (blocking), shapes must match.
void copy_accessor_data_to_l_from_r(GenericTensorAccessorW const &dst, GenericTensorAccessorR const &src);
void fill_with_zeros(GenericTensorAccessorW const &);

}  // namespace FlexFlow
