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

  // accessor.h:24-29: the typed pointer, after a check of the data type
  template <DataType DT>
  real_type_t<DT> const *get() const { return typed<real_type_t<DT>>(DT); }
  float const *get_float_ptr() const { return get<DataType::FLOAT>(); }
  double const *get_double_ptr() const { return get<DataType::DOUBLE>(); }
  half const *get_half_ptr() const { return get<DataType::HALF>(); }
  int32_t const *get_int32_ptr() const { return get<DataType::INT32>(); }
  int64_t const *get_int64_ptr() const { return get<DataType::INT64>(); }

  // accessor.h:46-57: element access on a CPU-resident accessor (residency and data type checked)
  template <DataType DT>
  real_type_t<DT> const &at(TensorDimsCoord const &coord) const {
    if (device_type != DeviceType::CPU) throw std::runtime_error("GenericTensorAccessorR::at() requires CPU-allocated tensor");
    return get<DT>()[calculate_accessor_offset(coord, shape.dims)];
  }
  // the same by element type (any type of the data type's size)
  template <typename T>
  T const &at(TensorDimsCoord const &coord) const {
    if (device_type != DeviceType::CPU) throw std::runtime_error("at() requires a CPU accessor");
    if (sizeof(T) != size_of_datatype(shape.data_type)) throw std::runtime_error("at(): dtype mismatch");
    return static_cast<T const *>(ptr)[calculate_accessor_offset(coord, shape.dims)];
  }

 private:
  template <typename T>
  T const *typed(DataType want) const {
    if (shape.data_type != want) throw std::runtime_error("accessor: Invalid datatype requested");
    return static_cast<T const *>(ptr);
  }
};

struct GenericTensorAccessorW {
  TensorShape shape;
  void *ptr;
  DeviceType device_type;

  operator GenericTensorAccessorR() const { return GenericTensorAccessorR{shape, ptr, device_type}; }
  template <DataType DT>
  real_type_t<DT> *get() const {
    if (shape.data_type != DT) throw std::runtime_error("accessor: Invalid datatype requested");
    return static_cast<real_type_t<DT> *>(ptr);
  }
  float *get_float_ptr() const { return get<DataType::FLOAT>(); }
  double *get_double_ptr() const { return get<DataType::DOUBLE>(); }
  half *get_half_ptr() const { return get<DataType::HALF>(); }
  int32_t *get_int32_ptr() const { return get<DataType::INT32>(); }
  int64_t *get_int64_ptr() const { return get<DataType::INT64>(); }
  template <DataType DT>
  real_type_t<DT> &at(TensorDimsCoord const &coord) const {
    if (device_type != DeviceType::CPU) throw std::runtime_error("GenericTensorAccessorW::at() requires CPU-allocated tensor");
    return get<DT>()[calculate_accessor_offset(coord, shape.dims)];
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
