// ComputationGraphBuilder: the operator methods models are written against
// (reference: lib/pcg/include/pcg/computation_graph_builder.h:17-330, bodies
// lib/pcg/src/pcg/computation_graph_builder.cc).  Each method adds the weight
// layers its operator needs, then the operator layer, and returns the output.
// Covered: the operators this library has kernels for.
#pragma once
#include "pcg/computation_graph.h"
#include <set>

namespace FlexFlow {

struct ComputationGraphBuilder {
  ComputationGraphBuilder();

  tensor_guid_t create_input(TensorShape const &, CreateGrad, std::optional<std::string> const &name = std::nullopt);
  tensor_guid_t create_weight(TensorShape const &, std::optional<std::string> const &name = std::nullopt);

  tensor_guid_t add(tensor_guid_t const &x, tensor_guid_t const &y, std::optional<std::string> const &name = std::nullopt);
  tensor_guid_t subtract(tensor_guid_t const &x, tensor_guid_t const &y, std::optional<std::string> const &name = std::nullopt);
  tensor_guid_t multiply(tensor_guid_t const &x, tensor_guid_t const &y, std::optional<std::string> const &name = std::nullopt);
  tensor_guid_t divide(tensor_guid_t const &x, tensor_guid_t const &y, std::optional<std::string> const &name = std::nullopt);
  tensor_guid_t max(tensor_guid_t const &x, tensor_guid_t const &y, std::optional<std::string> const &name = std::nullopt);
  tensor_guid_t min(tensor_guid_t const &x, tensor_guid_t const &y, std::optional<std::string> const &name = std::nullopt);

  tensor_guid_t exp(tensor_guid_t const &x, std::optional<std::string> const &name = std::nullopt);
  tensor_guid_t rsqrt(tensor_guid_t const &x, std::optional<std::string> const &name = std::nullopt);
  tensor_guid_t pow(tensor_guid_t const &x, float exponent, std::optional<std::string> const &name = std::nullopt);
  tensor_guid_t scalar_multiply(tensor_guid_t const &x, float scalar, std::optional<std::string> const &name = std::nullopt);
  tensor_guid_t scalar_add(tensor_guid_t const &x, float scalar, std::optional<std::string> const &name = std::nullopt);
  tensor_guid_t scalar_sub(tensor_guid_t const &x, float scalar, std::optional<std::string> const &name = std::nullopt);
  tensor_guid_t scalar_truediv(tensor_guid_t const &x, float scalar, std::optional<std::string> const &name = std::nullopt);
  tensor_guid_t sin(tensor_guid_t const &x, std::optional<std::string> const &name = std::nullopt);
  tensor_guid_t cos(tensor_guid_t const &x, std::optional<std::string> const &name = std::nullopt);
  tensor_guid_t relu(tensor_guid_t const &x, std::optional<std::string> const &name = std::nullopt);
  tensor_guid_t identity(tensor_guid_t const &x, std::optional<std::string> const &name = std::nullopt);
  tensor_guid_t gelu(tensor_guid_t const &x, std::optional<std::string> const &name = std::nullopt);
  tensor_guid_t sigmoid(tensor_guid_t const &x, std::optional<std::string> const &name = std::nullopt);
  tensor_guid_t tanh(tensor_guid_t const &x, std::optional<std::string> const &name = std::nullopt);
  tensor_guid_t elu(tensor_guid_t const &x, std::optional<std::string> const &name = std::nullopt);

  tensor_guid_t dropout(tensor_guid_t const &input, float rate, unsigned long long seed = 0,
                        std::optional<std::string> const &name = std::nullopt);
  tensor_guid_t embedding(tensor_guid_t const &input, int num_entries, int outDim, std::optional<AggregateOp> aggr,
                          DataType dtype = DataType::FLOAT, std::optional<std::string> const &name = std::nullopt);
  tensor_guid_t layer_norm(tensor_guid_t const &input, std::set<int> const &axes, bool elementwise_affine, float eps,
                           std::optional<std::string> const &name = std::nullopt);
  // Weights and output take the input's data type.
  tensor_guid_t dense(tensor_guid_t const &input, int outDim, std::optional<Activation> activation = std::nullopt,
                      bool use_bias = true, std::optional<std::string> const &name = std::nullopt);
  tensor_guid_t cast(tensor_guid_t const &input, DataType dtype, std::optional<std::string> const &name = std::nullopt);
  tensor_guid_t concat(std::vector<tensor_guid_t> const &tensors, int axis,
                       std::optional<std::string> const &name = std::nullopt);
  tensor_guid_t transpose(tensor_guid_t const &input, std::vector<int> const &perm,
                          std::optional<std::string> const &name = std::nullopt);
  tensor_guid_t reshape(tensor_guid_t const &input, std::vector<int64_t> const &shape,
                        std::optional<std::string> const &name = std::nullopt);
  tensor_guid_t gather(tensor_guid_t const &input, tensor_guid_t const &index, int dim,
                       std::optional<std::string> const &name = std::nullopt);
  tensor_guid_t softmax(tensor_guid_t const &input, std::optional<int> dim = std::nullopt,
                        std::optional<std::string> const &name = std::nullopt);
  // `scale` and `causal` extend the reference's signature (its kernel fixes 1.0 / false).
  tensor_guid_t multihead_attention(tensor_guid_t const &query, tensor_guid_t const &key, tensor_guid_t const &value,
                                    int embed_dim, int num_heads, std::optional<int> kdim = std::nullopt,
                                    std::optional<int> vdim = std::nullopt, float dropout = 0.0f, bool bias = true,
                                    bool add_bias_kv = false, bool add_zero_attn = false,
                                    std::optional<std::string> const &name = std::nullopt, float scale = 1.0f,
                                    bool causal = false);

  TensorShape get_shape(tensor_guid_t const &) const;
  // the weight tensors of the layer that produced `output` (in the operator's weight order)
  std::vector<tensor_guid_t> get_weights_of(tensor_guid_t const &output) const;

  ComputationGraph computation_graph;

 private:
  tensor_guid_t add_op(ComputationGraphOpAttrs const &attrs, std::vector<tensor_guid_t> const &inputs,
                       std::optional<std::string> const &name);
  tensor_guid_t element_unary(OperatorType, tensor_guid_t const &, std::optional<float> scalar,
                              std::optional<std::string> const &name);
  tensor_guid_t element_binary(OperatorType, tensor_guid_t const &, tensor_guid_t const &,
                               std::optional<std::string> const &name);
};

}  // namespace FlexFlow
