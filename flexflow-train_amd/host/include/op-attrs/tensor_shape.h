// TensorDims / TensorShape / ff_dim_t (reference:
// lib/op-attrs/include/op-attrs/tensor_dims.dtg.toml, tensor_shape.dtg.toml,
// ff_dim_t.dtg.toml).  Dims are in FF order: dim 0 outermost.
#pragma once
#include "op-attrs/datatype.h"
#include <cstdint>
#include <vector>

namespace FlexFlow {

struct ff_dim_t {
  int value;
  bool operator==(ff_dim_t const &o) const { return value == o.value; }
};

using num_tensor_dims_t = int;

struct TensorDims {
  std::vector<int64_t> ff_ordered;
  bool operator==(TensorDims const &o) const { return ff_ordered == o.ff_ordered; }
  bool operator!=(TensorDims const &o) const { return !(*this == o); }
};

struct TensorShape {
  TensorDims dims;
  DataType data_type;
  bool operator==(TensorShape const &o) const { return dims == o.dims && data_type == o.data_type; }
  bool operator!=(TensorShape const &o) const { return !(*this == o); }
};

inline int get_num_dims(TensorDims const &d) { return (int)d.ff_ordered.size(); }
inline int64_t dim_at_idx(TensorDims const &d, int idx) {
  int n = (int)d.ff_ordered.size();
  return d.ff_ordered.at(idx < 0 ? n + idx : idx);  // negative = from the end
}
inline int64_t get_num_elements(TensorDims const &d) {
  int64_t n = 1;
  for (int64_t v : d.ff_ordered) n *= v;
  return n;
}
// True when `operand` lines up with the trailing dims of `out` once its leading
// 1s are dropped: the only broadcast the element-wise kernels implement (the
// smaller operand repeats every get_num_elements(operand) elements).  A size-1
// dim in the middle or at the end of the operand is a different pattern.
inline bool broadcasts_over_leading_dims(TensorDims const &operand, TensorDims const &out) {
  size_t first = 0;
  while (first < operand.ff_ordered.size() && operand.ff_ordered[first] == 1) first++;
  size_t const n = operand.ff_ordered.size() - first, m = out.ff_ordered.size();
  if (n > m) return false;
  for (size_t i = 0; i < n; i++) {
    if (operand.ff_ordered[first + i] != out.ff_ordered[m - n + i]) return false;
  }
  return true;
}
inline int64_t get_size_in_bytes(TensorShape const &s) {
  return get_num_elements(s.dims) * (int64_t)size_of_datatype(s.data_type);
}

}  // namespace FlexFlow
