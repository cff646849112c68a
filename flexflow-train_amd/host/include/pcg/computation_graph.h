// ComputationGraph: the layer list a training step is built from (reference:
// lib/pcg/include/pcg/computation_graph.h, layer_attrs.dtg.toml,
// lib/op-attrs/include/op-attrs/computation_graph_op_attrs.dtg.toml and the
// per-op attrs under lib/op-attrs/include/op-attrs/ops/).  Layers can only
// consume tensors that already exist, so insertion order is a topological
// order; no graph library is needed behind it.
#pragma once
#include "op-attrs/attrs.h"
#include "op-attrs/tensor_shape.h"
#include <functional>
#include <optional>
#include <string>
#include <variant>
#include <vector>

namespace FlexFlow {

struct tensor_guid_t {
  int raw;
  bool operator==(tensor_guid_t const &o) const { return raw == o.raw; }
  bool operator!=(tensor_guid_t const &o) const { return raw != o.raw; }
  bool operator<(tensor_guid_t const &o) const { return raw < o.raw; }
};
struct layer_guid_t {
  int raw;
  bool operator==(layer_guid_t const &o) const { return raw == o.raw; }
  bool operator!=(layer_guid_t const &o) const { return raw != o.raw; }
  bool operator<(layer_guid_t const &o) const { return raw < o.raw; }
};

enum class CreateGrad { YES, NO };

struct InputAttrs { TensorShape tensor_shape; };
// The initializer of the reference's WeightAttrs is left out: local execution
// never runs it (tensor_allocation.cc:35-49 allocates and nothing fills).
struct WeightAttrs { TensorShape tensor_shape; };
struct LayerNormAttrs {
  std::vector<int> axes;  // relative dims (negative = from the end); must be the trailing dims
  bool elementwise_affine;
  float eps;
};
struct MultiHeadAttentionAttrs {
  int embed_dim, num_heads, kdim, vdim;
  float dropout;  // ignored by the kernels, as in attention_kernels.cu:80-81
  bool bias, add_bias_kv, add_zero_attn;
  float scale = 1.0f;   // the reference's smScalar (attention_kernels.cu:76)
  bool causal = false;
};
struct ElementBinaryAttrs {
  OperatorType type;
  DataType compute_type;
  bool should_broadcast_lhs, should_broadcast_rhs;
};
struct SoftmaxAttrs { int dim; };  // relative dim
struct EmbeddingAttrs {
  int num_entries, out_channels;
  std::optional<AggregateOp> aggr;
  DataType data_type;
};
struct CastAttrs { DataType dtype; };
struct ConcatAttrs { int axis; };  // relative dim
struct ReshapeAttrs { TensorDims shape; };
struct GatherAttrs { int dim; };  // relative dim; inputs: values, index

using ComputationGraphOpAttrs =
    std::variant<InputAttrs, WeightAttrs, LinearAttrs, LayerNormAttrs, MultiHeadAttentionAttrs, DropoutAttrs,
                 ElementUnaryAttrs, ElementBinaryAttrs, SoftmaxAttrs, EmbeddingAttrs, CastAttrs, ConcatAttrs, TransposeAttrs, ReshapeAttrs,
                 GatherAttrs>;

struct LayerAttrs {
  ComputationGraphOpAttrs op_attrs;
  std::optional<std::string> name;
};

struct ComputationGraph {
  struct Layer {
    LayerAttrs attrs;
    std::vector<tensor_guid_t> inputs, weights, outputs;
  };
  struct Tensor {
    TensorShape shape;
    CreateGrad create_grad;
    layer_guid_t source;
  };
  std::vector<Layer> layers;
  std::vector<Tensor> tensors;
};

struct LayerAddedResult {
  layer_guid_t layer;
  std::vector<tensor_guid_t> outputs;
};

ComputationGraph make_empty_computation_graph();
// Output shapes are inferred from the attrs and the input shapes; weight
// tensors must have the shapes get_weight_shapes() names.
LayerAddedResult add_layer(ComputationGraph &cg, LayerAttrs const &attrs,
                           std::vector<tensor_guid_t> const &inputs,
                           std::vector<tensor_guid_t> const &weights);
LayerAddedResult add_input_layer(ComputationGraph &cg, TensorShape const &shape);
LayerAddedResult add_input_layer_with_grad(ComputationGraph &cg, TensorShape const &shape);
LayerAddedResult add_weight_layer(ComputationGraph &cg, TensorShape const &shape);

TensorShape get_tensor_shape(ComputationGraph const &cg, tensor_guid_t t);
std::vector<TensorShape> get_output_shapes(ComputationGraphOpAttrs const &attrs,
                                           std::vector<TensorShape> const &input_shapes);
std::vector<TensorShape> get_weight_shapes(ComputationGraphOpAttrs const &attrs,
                                           std::vector<TensorShape> const &input_shapes);
std::vector<layer_guid_t> topological_ordering(ComputationGraph const &cg);
bool are_tensor_guid_shapes_equivalent(ComputationGraph const &cg, tensor_guid_t a, tensor_guid_t b);

}  // namespace FlexFlow

namespace std {
template <> struct hash<FlexFlow::tensor_guid_t> {
  size_t operator()(FlexFlow::tensor_guid_t const &t) const noexcept { return std::hash<int>()(t.raw); }
};
template <> struct hash<FlexFlow::layer_guid_t> {
  size_t operator()(FlexFlow::layer_guid_t const &l) const noexcept { return std::hash<int>()(l.raw); }
};
}  // namespace std
