// Operator attribute value types that appear on the kernel signatures.  Field
// names and order follow the reference's generated structs:
//   Activation        lib/op-attrs/include/op-attrs/activation.dtg.toml
//   AggregateOp       lib/op-attrs/include/op-attrs/aggregate_op.dtg.toml
//   RegularizerAttrs  lib/op-attrs/include/op-attrs/regularizer_attrs.dtg.toml
//   OperatorType      lib/op-attrs/include/op-attrs/operator_type.dtg.toml:12-94
//   LinearAttrs       lib/op-attrs/include/op-attrs/ops/linear_attrs.dtg.toml:32-50
//   ElementUnaryAttrs lib/op-attrs/include/op-attrs/ops/element_unary_attrs.dtg.toml
//   DropoutAttrs      lib/op-attrs/include/op-attrs/ops/dropout_attrs.dtg.toml
//   TransposeAttrs    lib/op-attrs/include/op-attrs/ops/transpose_attrs.dtg.toml
#pragma once
#include "op-attrs/datatype.h"
#include <optional>
#include <variant>
#include <vector>

namespace FlexFlow {

enum class Activation { RELU, SIGMOID, TANH, GELU };
enum class AggregateOp { SUM, AVG };

struct L1RegularizerAttrs { float lambda; };
struct L2RegularizerAttrs { float lambda; };
using RegularizerAttrs = std::variant<L1RegularizerAttrs, L2RegularizerAttrs>;

enum class OperatorType {
  NOOP, INPUT, WEIGHT, CONV2D, DROPOUT, LINEAR, BATCHMATMUL, POOL2D, SCALAR_MULTIPLY,
  SCALAR_ADD, SCALAR_FLOOR_DIV, SCALAR_TRUE_DIV, SCALAR_SUB, RELU, IDENTITY, SIGMOID, TANH,
  ELU, FLAT, SOFTMAX, BATCHNORM, CONCAT, SPLIT, EMBEDDING, CACHE, RESHAPE, REVERSE,
  TRANSPOSE, EW_ADD, EW_MUL, MATMUL, MUL, ENLARGE, SQUEEZE, UNSQUEEZE, EW_SUB, EW_DIV,
  EW_EQUAL, EW_GREATER, EW_LESS, EW_MAX, EW_MIN, REDUCE_ARGMAX, REDUCE_ARGMIN, REDUCE_MAX,
  REDUCE_MEAN, REDUCE_MIN, REDUCE_PROD, REDUCE_SUM, PAD, SHAPE, SIZE, TOPK, WHERE, CEIL,
  CAST, EXP, ROUND, LOG, LOGICAL_NOT, SQRT, SIN, COS, LEAKYRELU, SLICE, RESIZE, PRELU, GELU,
  MULTIHEAD_ATTENTION, FUSED, RSQRT, POW, MEAN, LAYERNORM, GATHER, BROADCAST, REPARTITION,
  COMBINE, REPLICATE, REDUCTION, BATCH, PIPELINE, FUSED_PARALLEL
};
static_assert(static_cast<int>(OperatorType::GELU) == 67, "ordinals must match the C ABI");
static_assert(static_cast<int>(OperatorType::EW_ADD) == 28, "ordinals must match the C ABI");
static_assert(static_cast<int>(OperatorType::POW) == 71, "ordinals must match the C ABI");

struct LinearAttrs {
  int out_channels;
  bool use_bias;
  DataType data_type;
  std::optional<Activation> activation;
  std::optional<RegularizerAttrs> regularizer;
};

struct ElementUnaryAttrs {
  OperatorType op_type;
  std::optional<float> scalar;
};

// output dim i is input dim permutation[i] (FF order)
struct TransposeAttrs {
  std::vector<int> permutation;
};

struct DropoutAttrs {
  float rate;
  unsigned long long seed;
};

}  // namespace FlexFlow
