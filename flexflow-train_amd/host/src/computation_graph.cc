// ComputationGraph, shape inference and ComputationGraphBuilder (reference:
// lib/pcg/src/pcg/computation_graph.cc, computation_graph_builder.cc and the
// get_output_shape / get_weights_shape functions under
// lib/op-attrs/src/op-attrs/ops/).
#include "ffk.h"
#include "pcg/computation_graph.h"
#include "pcg/computation_graph_builder.h"
#include <stdexcept>

namespace FlexFlow {

[[noreturn]] static void bad(std::string const &msg) { throw std::runtime_error("computation graph: " + msg); }

static bool is_integer(DataType d) { return d == DataType::INT32 || d == DataType::INT64; }

static int64_t trailing_extent(TensorShape const &s, std::vector<int> const &axes) {
  // the normalised axes must be exactly the last axes.size() dims
  int nd = get_num_dims(s.dims);
  std::vector<bool> hit(nd, false);
  for (int a : axes) {
    int i = a < 0 ? nd + a : a;
    if (i < 0 || i >= nd) bad("LayerNorm axis out of range");
    hit[i] = true;
  }
  int64_t n = 1;
  int count = 0;
  for (int i = nd - 1; i >= 0 && hit[i]; i--) {
    n *= s.dims.ff_ordered[i];
    count++;
  }
  if (count != (int)axes.size() || count == 0) bad("LayerNorm normalises trailing dims only");
  return n;
}

static int64_t mha_weight_elements(MultiHeadAttentionAttrs const &a, std::vector<TensorShape> const &in) {
  ffk_mha_desc_t d{};
  d.num_samples = dim_at_idx(in[0].dims, 0);
  d.num_heads = a.num_heads;
  d.q_size = dim_at_idx(in[0].dims, -1);
  d.k_size = dim_at_idx(in[1].dims, -1);
  d.v_size = dim_at_idx(in[2].dims, -1);
  d.q_proj_size = a.kdim;
  d.k_proj_size = a.kdim;
  d.v_proj_size = a.vdim;
  d.o_proj_size = a.embed_dim;
  d.qo_seq_length = dim_at_idx(in[0].dims, 1);
  d.kv_seq_length = dim_at_idx(in[1].dims, 1);
  d.scale = a.scale;
  d.causal = a.causal;
  return (int64_t)ffk_mha_weight_elements(&d);
}

std::vector<TensorShape> get_output_shapes(ComputationGraphOpAttrs const &attrs, std::vector<TensorShape> const &in) {
  auto need = [&](size_t n) {
    if (in.size() != n) bad("operator expects " + std::to_string(n) + " inputs");
  };
  if (auto const *a = std::get_if<InputAttrs>(&attrs)) {
    need(0);
    return {a->tensor_shape};
  }
  if (auto const *a = std::get_if<WeightAttrs>(&attrs)) {
    need(0);
    return {a->tensor_shape};
  }
  if (auto const *a = std::get_if<LinearAttrs>(&attrs)) {
    // linear.cc: last dim -> out_channels
    need(1);
    TensorShape o = in[0];
    o.dims.ff_ordered.back() = a->out_channels;
    return {o};
  }
  if (auto const *a = std::get_if<LayerNormAttrs>(&attrs)) {
    need(1);
    (void)trailing_extent(in[0], a->axes);
    return {in[0]};
  }
  if (auto const *a = std::get_if<MultiHeadAttentionAttrs>(&attrs)) {
    // attention.cc: [batch, seq_q, embed_dim]
    need(3);
    for (auto const &s : in) {
      if (get_num_dims(s.dims) != 3) bad("attention inputs are [batch, seq, size]");
    }
    if (in[1].dims.ff_ordered[1] != in[2].dims.ff_ordered[1] || in[0].dims.ff_ordered[0] != in[1].dims.ff_ordered[0] ||
        in[0].dims.ff_ordered[0] != in[2].dims.ff_ordered[0]) {
      bad("attention: key/value sequence lengths or batch sizes differ");
    }
    return {TensorShape{TensorDims{{in[0].dims.ff_ordered[0], in[0].dims.ff_ordered[1], (int64_t)a->embed_dim}},
                        in[0].data_type}};
  }
  if (std::get_if<DropoutAttrs>(&attrs) || std::get_if<ElementUnaryAttrs>(&attrs)) {
    need(1);
    return {in[0]};
  }
  if (std::get_if<ElementBinaryAttrs>(&attrs)) {
    need(2);
    if (in[0].data_type != in[1].data_type) bad("element binary: operand data types differ");
    int64_t nl = get_num_elements(in[0].dims), nr = get_num_elements(in[1].dims);
    TensorShape const &big = nl >= nr ? in[0] : in[1];
    int64_t small = nl >= nr ? nr : nl;
    if (get_num_elements(big.dims) % small != 0) bad("element binary: operand does not broadcast over trailing dims");
    TensorShape const &little = nl >= nr ? in[1] : in[0];
    if (!broadcasts_over_leading_dims(little.dims, big.dims)) {
      bad("element binary: broadcast pattern not supported (the smaller operand must equal the output's trailing dims)");
    }
    return {big};
  }
  if (auto const *a = std::get_if<SoftmaxAttrs>(&attrs)) {
    need(1);
    int nd = get_num_dims(in[0].dims);
    int d = a->dim < 0 ? nd + a->dim : a->dim;
    if (d < 0 || d >= nd) bad("softmax dim out of range");
    return {in[0]};
  }
  if (auto const *a = std::get_if<EmbeddingAttrs>(&attrs)) {
    // embedding.cc:31-36: the last input dim becomes out_channels; without an
    // aggregation every index keeps its own row, so out_channels is appended
    need(1);
    if (!is_integer(in[0].data_type)) bad("embedding expects INT32 or INT64 indices");
    TensorShape o = in[0];
    if (a->aggr.has_value()) {
      o.dims.ff_ordered.back() = a->out_channels;
    } else {
      o.dims.ff_ordered.push_back(a->out_channels);
    }
    o.data_type = a->data_type;
    return {o};
  }
  if (auto const *a = std::get_if<ConcatAttrs>(&attrs)) {
    // concat.cc: equal shapes outside the axis, extents add along it
    if (in.empty()) bad("concat expects at least one input");
    int nd = get_num_dims(in[0].dims);
    int axis = a->axis < 0 ? nd + a->axis : a->axis;
    if (axis < 0 || axis >= nd) bad("concat axis out of range");
    TensorShape o = in[0];
    o.dims.ff_ordered[axis] = 0;
    for (TensorShape const &s : in) {
      if (s.data_type != in[0].data_type || get_num_dims(s.dims) != nd) bad("concat: inputs differ in data type or rank");
      for (int i = 0; i < nd; i++) {
        if (i != axis && s.dims.ff_ordered[i] != in[0].dims.ff_ordered[i]) bad("concat: shapes differ outside the axis");
      }
      o.dims.ff_ordered[axis] += s.dims.ff_ordered[axis];
    }
    return {o};
  }
  if (auto const *a = std::get_if<TransposeAttrs>(&attrs)) {
    need(1);
    int nd = get_num_dims(in[0].dims);
    if ((int)a->permutation.size() != nd) bad("transpose: permutation length differs from the rank");
    std::vector<bool> seen(nd, false);
    TensorShape o = in[0];
    for (int i = 0; i < nd; i++) {
      int p = a->permutation[i];
      if (p < 0 || p >= nd || seen[p]) bad("transpose: not a permutation");
      seen[p] = true;
      o.dims.ff_ordered[i] = in[0].dims.ff_ordered[p];
    }
    return {o};
  }
  if (auto const *a = std::get_if<ReshapeAttrs>(&attrs)) {
    need(1);
    if (get_num_elements(a->shape) != get_num_elements(in[0].dims)) bad("reshape: element counts differ");
    return {TensorShape{a->shape, in[0].data_type}};
  }
  if (auto const *a = std::get_if<GatherAttrs>(&attrs)) {
    // gather.cc: the output takes the index's dims and the values' data type
    need(2);
    if (!is_integer(in[1].data_type)) bad("gather expects INT32 or INT64 indices");
    int nd = get_num_dims(in[0].dims);
    int d = a->dim < 0 ? nd + a->dim : a->dim;
    if (d < 0 || d >= nd || get_num_dims(in[1].dims) != nd) bad("gather: dim or ranks out of range");
    for (int i = 0; i < nd; i++) {
      if (i != d && in[0].dims.ff_ordered[i] != in[1].dims.ff_ordered[i]) bad("gather: shapes differ outside the dim");
    }
    return {TensorShape{in[1].dims, in[0].data_type}};
  }
  if (auto const *a = std::get_if<CastAttrs>(&attrs)) {
    need(1);
    TensorShape o = in[0];
    o.data_type = a->dtype;
    return {o};
  }
  bad("unknown operator");
}

std::vector<TensorShape> get_weight_shapes(ComputationGraphOpAttrs const &attrs, std::vector<TensorShape> const &in) {
  if (auto const *a = std::get_if<LinearAttrs>(&attrs)) {
    // projection [out_channels, in_channels], bias [out_channels] (linear.cc)
    std::vector<TensorShape> w = {
        TensorShape{TensorDims{{(int64_t)a->out_channels, in.at(0).dims.ff_ordered.back()}}, in[0].data_type}};
    if (a->use_bias) w.push_back(TensorShape{TensorDims{{(int64_t)a->out_channels}}, in[0].data_type});
    return w;
  }
  if (auto const *a = std::get_if<LayerNormAttrs>(&attrs)) {
    // gamma and beta over the normalised extent, which is how the kernel
    // indexes them (layer_norm_kernels.cu:104-107)
    if (!a->elementwise_affine) return {};
    int64_t n = trailing_extent(in.at(0), a->axes);
    TensorShape s{TensorDims{{n}}, in[0].data_type};
    return {s, s};
  }
  if (auto const *a = std::get_if<MultiHeadAttentionAttrs>(&attrs)) {
    return {TensorShape{TensorDims{{mha_weight_elements(*a, in)}}, in.at(0).data_type}};
  }
  if (auto const *a = std::get_if<EmbeddingAttrs>(&attrs)) {
    // fp32 table: the scatter-add accumulates in fp32
    return {TensorShape{TensorDims{{(int64_t)a->num_entries, (int64_t)a->out_channels}}, DataType::FLOAT}};
  }
  return {};
}

ComputationGraph make_empty_computation_graph() { return ComputationGraph{}; }

TensorShape get_tensor_shape(ComputationGraph const &cg, tensor_guid_t t) { return cg.tensors.at(t.raw).shape; }

bool are_tensor_guid_shapes_equivalent(ComputationGraph const &cg, tensor_guid_t a, tensor_guid_t b) {
  return get_tensor_shape(cg, a) == get_tensor_shape(cg, b);
}

static LayerAddedResult add_layer_with_grad(ComputationGraph &cg, LayerAttrs const &attrs,
                                            std::vector<tensor_guid_t> const &inputs,
                                            std::vector<tensor_guid_t> const &weights, CreateGrad create_grad) {
  std::vector<TensorShape> in_shapes;
  for (tensor_guid_t t : inputs) in_shapes.push_back(get_tensor_shape(cg, t));
  std::vector<TensorShape> want = get_weight_shapes(attrs.op_attrs, in_shapes);
  if (want.size() != weights.size()) bad("operator expects " + std::to_string(want.size()) + " weight tensors");
  for (size_t i = 0; i < want.size(); i++) {
    if (get_tensor_shape(cg, weights[i]) != want[i]) bad("weight tensor " + std::to_string(i) + " has the wrong shape");
    if (!std::holds_alternative<WeightAttrs>(cg.layers.at(cg.tensors.at(weights[i].raw).source.raw).attrs.op_attrs)) {
      bad("weight slot is not fed by a weight layer");
    }
  }
  layer_guid_t id{(int)cg.layers.size()};
  ComputationGraph::Layer layer{attrs, inputs, weights, {}};
  for (TensorShape const &s : get_output_shapes(attrs.op_attrs, in_shapes)) {
    layer.outputs.push_back(tensor_guid_t{(int)cg.tensors.size()});
    cg.tensors.push_back(ComputationGraph::Tensor{s, create_grad, id});
  }
  cg.layers.push_back(layer);
  return LayerAddedResult{id, layer.outputs};
}

LayerAddedResult add_layer(ComputationGraph &cg, LayerAttrs const &attrs, std::vector<tensor_guid_t> const &inputs,
                           std::vector<tensor_guid_t> const &weights) {
  return add_layer_with_grad(cg, attrs, inputs, weights, CreateGrad::YES);
}
LayerAddedResult add_input_layer(ComputationGraph &cg, TensorShape const &shape) {
  return add_layer_with_grad(cg, LayerAttrs{InputAttrs{shape}, std::nullopt}, {}, {}, CreateGrad::NO);
}
LayerAddedResult add_input_layer_with_grad(ComputationGraph &cg, TensorShape const &shape) {
  return add_layer_with_grad(cg, LayerAttrs{InputAttrs{shape}, std::nullopt}, {}, {}, CreateGrad::YES);
}
LayerAddedResult add_weight_layer(ComputationGraph &cg, TensorShape const &shape) {
  return add_layer_with_grad(cg, LayerAttrs{WeightAttrs{shape}, std::nullopt}, {}, {}, CreateGrad::YES);
}

std::vector<layer_guid_t> topological_ordering(ComputationGraph const &cg) {
  std::vector<layer_guid_t> order;
  for (size_t i = 0; i < cg.layers.size(); i++) order.push_back(layer_guid_t{(int)i});
  return order;
}

// ---- builder ----------------------------------------------------------------

ComputationGraphBuilder::ComputationGraphBuilder() : computation_graph(make_empty_computation_graph()) {}

tensor_guid_t ComputationGraphBuilder::create_input(TensorShape const &shape, CreateGrad g,
                                                    std::optional<std::string> const &name) {
  LayerAddedResult r = g == CreateGrad::YES ? add_input_layer_with_grad(computation_graph, shape)
                                            : add_input_layer(computation_graph, shape);
  computation_graph.layers[r.layer.raw].attrs.name = name;
  return r.outputs.at(0);
}

tensor_guid_t ComputationGraphBuilder::create_weight(TensorShape const &shape, std::optional<std::string> const &name) {
  LayerAddedResult r = add_weight_layer(computation_graph, shape);
  computation_graph.layers[r.layer.raw].attrs.name = name;
  return r.outputs.at(0);
}

tensor_guid_t ComputationGraphBuilder::add_op(ComputationGraphOpAttrs const &attrs,
                                              std::vector<tensor_guid_t> const &inputs,
                                              std::optional<std::string> const &name) {
  std::vector<TensorShape> in_shapes;
  for (tensor_guid_t t : inputs) in_shapes.push_back(get_shape(t));
  std::vector<tensor_guid_t> weights;
  for (TensorShape const &s : get_weight_shapes(attrs, in_shapes)) weights.push_back(create_weight(s));
  return add_layer(computation_graph, LayerAttrs{attrs, name}, inputs, weights).outputs.at(0);
}

TensorShape ComputationGraphBuilder::get_shape(tensor_guid_t const &t) const {
  return get_tensor_shape(computation_graph, t);
}

std::vector<tensor_guid_t> ComputationGraphBuilder::get_weights_of(tensor_guid_t const &output) const {
  return computation_graph.layers.at(computation_graph.tensors.at(output.raw).source.raw).weights;
}

tensor_guid_t ComputationGraphBuilder::element_unary(OperatorType op, tensor_guid_t const &x, std::optional<float> scalar,
                                                     std::optional<std::string> const &name) {
  return add_op(ElementUnaryAttrs{op, scalar}, {x}, name);
}
tensor_guid_t ComputationGraphBuilder::element_binary(OperatorType op, tensor_guid_t const &x, tensor_guid_t const &y,
                                                      std::optional<std::string> const &name) {
  int64_t nl = get_num_elements(get_shape(x).dims), nr = get_num_elements(get_shape(y).dims);
  return add_op(ElementBinaryAttrs{op, get_shape(x).data_type, nl < nr, nr < nl}, {x, y}, name);
}

#define FFK_BINARY(method, OP)                                                                           \
  tensor_guid_t ComputationGraphBuilder::method(tensor_guid_t const &x, tensor_guid_t const &y,         \
                                                std::optional<std::string> const &name) {               \
    return element_binary(OperatorType::OP, x, y, name);                                                 \
  }
FFK_BINARY(add, EW_ADD)
FFK_BINARY(subtract, EW_SUB)
FFK_BINARY(multiply, EW_MUL)
FFK_BINARY(divide, EW_DIV)
FFK_BINARY(max, EW_MAX)
FFK_BINARY(min, EW_MIN)
#undef FFK_BINARY

#define FFK_UNARY(method, OP)                                                                            \
  tensor_guid_t ComputationGraphBuilder::method(tensor_guid_t const &x, std::optional<std::string> const &name) { \
    return element_unary(OperatorType::OP, x, std::nullopt, name);                                       \
  }
FFK_UNARY(exp, EXP)
FFK_UNARY(rsqrt, RSQRT)
FFK_UNARY(sin, SIN)
FFK_UNARY(cos, COS)
FFK_UNARY(relu, RELU)
FFK_UNARY(identity, IDENTITY)
FFK_UNARY(gelu, GELU)
FFK_UNARY(sigmoid, SIGMOID)
FFK_UNARY(tanh, TANH)
FFK_UNARY(elu, ELU)
#undef FFK_UNARY

#define FFK_SCALAR(method, OP)                                                                           \
  tensor_guid_t ComputationGraphBuilder::method(tensor_guid_t const &x, float scalar,                    \
                                                std::optional<std::string> const &name) {               \
    return element_unary(OperatorType::OP, x, scalar, name);                                             \
  }
FFK_SCALAR(pow, POW)
FFK_SCALAR(scalar_multiply, SCALAR_MULTIPLY)
FFK_SCALAR(scalar_add, SCALAR_ADD)
FFK_SCALAR(scalar_sub, SCALAR_SUB)
FFK_SCALAR(scalar_truediv, SCALAR_TRUE_DIV)
#undef FFK_SCALAR

tensor_guid_t ComputationGraphBuilder::dropout(tensor_guid_t const &input, float rate, unsigned long long seed,
                                               std::optional<std::string> const &name) {
  return add_op(DropoutAttrs{rate, seed}, {input}, name);
}
tensor_guid_t ComputationGraphBuilder::embedding(tensor_guid_t const &input, int num_entries, int outDim,
                                                 std::optional<AggregateOp> aggr, DataType dtype,
                                                 std::optional<std::string> const &name) {
  return add_op(EmbeddingAttrs{num_entries, outDim, aggr, dtype}, {input}, name);
}
tensor_guid_t ComputationGraphBuilder::layer_norm(tensor_guid_t const &input, std::set<int> const &axes,
                                                  bool elementwise_affine, float eps,
                                                  std::optional<std::string> const &name) {
  return add_op(LayerNormAttrs{std::vector<int>(axes.begin(), axes.end()), elementwise_affine, eps}, {input}, name);
}
tensor_guid_t ComputationGraphBuilder::dense(tensor_guid_t const &input, int outDim, std::optional<Activation> activation,
                                             bool use_bias, std::optional<std::string> const &name) {
  // Linear's backward has no GELU (like the reference's, linear_kernels.cu:228-244, it would
  // need the pre-activation), so that activation becomes its own ElementUnary layer.
  if (activation.has_value() && *activation == Activation::GELU) {
    tensor_guid_t pre = add_op(LinearAttrs{outDim, use_bias, get_shape(input).data_type, std::nullopt, std::nullopt}, {input}, name);
    return gelu(pre);
  }
  return add_op(LinearAttrs{outDim, use_bias, get_shape(input).data_type, activation, std::nullopt}, {input}, name);
}
tensor_guid_t ComputationGraphBuilder::cast(tensor_guid_t const &input, DataType dtype,
                                            std::optional<std::string> const &name) {
  return add_op(CastAttrs{dtype}, {input}, name);
}
tensor_guid_t ComputationGraphBuilder::concat(std::vector<tensor_guid_t> const &tensors, int axis,
                                              std::optional<std::string> const &name) {
  return add_op(ConcatAttrs{axis}, tensors, name);
}
tensor_guid_t ComputationGraphBuilder::transpose(tensor_guid_t const &input, std::vector<int> const &perm,
                                                 std::optional<std::string> const &name) {
  return add_op(TransposeAttrs{perm}, {input}, name);
}
tensor_guid_t ComputationGraphBuilder::reshape(tensor_guid_t const &input, std::vector<int64_t> const &shape,
                                               std::optional<std::string> const &name) {
  return add_op(ReshapeAttrs{TensorDims{shape}}, {input}, name);
}
tensor_guid_t ComputationGraphBuilder::gather(tensor_guid_t const &input, tensor_guid_t const &index, int dim,
                                              std::optional<std::string> const &name) {
  return add_op(GatherAttrs{dim}, {input, index}, name);
}
tensor_guid_t ComputationGraphBuilder::softmax(tensor_guid_t const &input, std::optional<int> dim,
                                               std::optional<std::string> const &name) {
  return add_op(SoftmaxAttrs{dim.value_or(-1)}, {input}, name);
}
tensor_guid_t ComputationGraphBuilder::multihead_attention(tensor_guid_t const &query, tensor_guid_t const &key,
                                                           tensor_guid_t const &value, int embed_dim, int num_heads,
                                                           std::optional<int> kdim, std::optional<int> vdim,
                                                           float dropout, bool bias, bool add_bias_kv,
                                                           bool add_zero_attn, std::optional<std::string> const &name,
                                                           float scale, bool causal) {
  // computation_graph_builder.cc: kdim / vdim default to embed_dim; the kernels take no bias
  if (add_bias_kv || add_zero_attn) bad("multihead_attention: add_bias_kv / add_zero_attn are not supported");
  MultiHeadAttentionAttrs a{embed_dim, num_heads, kdim.value_or(embed_dim), vdim.value_or(embed_dim), dropout,
                            bias,      add_bias_kv, add_zero_attn,           scale,                      causal};
  return add_op(a, {query, key, value}, name);
}

}  // namespace FlexFlow
