// The training-step driver (reference: lib/local-execution/src/local-execution/
// computation_graph_instance.cc:61-260, task_execution.cc:84-125,
// tensor_allocation.cc, per_device_op_state_initialization.cc:21-56; the task
// bodies it dispatches to are lib/task-spec/src/task-spec/ops/impl/*.cc,
// loss_functions.cc:24-150 and optimizer.cc:10-108).
//
// Everything a step needs is decided once, here: one device allocation holds
// every tensor the caller did not bring (gradients that are added into first,
// so a single fill clears them), the saved operator state and a scratch region
// the backward kernels share; each invocation is a closure over final device
// pointers that makes one C-ABI call.
#include "ffk.h"
#include "local-execution/computation_graph_instance.h"
#include <memory>
#include <cstdlib>
#include <cmath>
#include <cstring>

namespace FlexFlow {

[[noreturn]] static void bad(std::string const &msg) { throw std::runtime_error("computation graph instance: " + msg); }

static int dt(DataType d) { return static_cast<int>(d); }
static bool is_float_type(DataType d) {
  return d == DataType::FLOAT || d == DataType::BF16 || d == DataType::HALF || d == DataType::DOUBLE;
}
static size_t align_up(size_t n) { return (n + 255) & ~(size_t)255; }

LossFunction get_loss_function(LossAttrs const &a) {
  if (std::holds_alternative<SparseCategoricalCrossEntropyLossAttrs>(a)) {
    return LossFunction::SPARSE_CATEGORICAL_CROSSENTROPY;
  }
  return std::get<NonconfigurableLossAttrs>(a).loss_type;
}

OptimizerAttrs get_optimizer_attrs_for_next_iter(OptimizerAttrs const &old_attrs) {
  if (auto const *old = std::get_if<AdamOptimizerAttrs>(&old_attrs)) {
    double new_beta1_t = old->beta_t * old->beta1;
    double new_beta2_t = old->beta2_t * old->beta2;
    double new_alpha_t = old->alpha * std::sqrt(1 - new_beta2_t) / (1 - new_beta1_t);
    return AdamOptimizerAttrs{old->alpha,  old->beta1,  old->beta2,  old->weight_decay,
                              new_alpha_t, new_beta1_t, new_beta2_t, old->epsilon};
  }
  return old_attrs;
}

// ---- state --------------------------------------------------------------------

struct ComputationGraphInstance::State {
  ComputationGraph cg;
  Allocator allocator;
  OptimizerAttrs optimizer_attrs;
  std::vector<GenericTensorAccessorW> value;
  std::vector<std::optional<GenericTensorAccessorW>> grad, master, opt_v, opt_m;
  std::optional<tensor_guid_t> logit;
  std::vector<DynamicNodeInvocation> order;
  char *arena = nullptr;
  size_t arena_bytes = 0, cleared_bytes = 0;
  bool masters_valid = false;
  uint64_t iteration = 0;

  State(ComputationGraph const &g, Allocator const &a, OptimizerAttrs const &o) : cg(g), allocator(a), optimizer_attrs(o) {}
  State(State const &) = delete;
  State &operator=(State const &) = delete;
  ~State() {
    if (arena != nullptr) allocator.deallocate(arena);
  }
};

ComputationGraphInstance::ComputationGraphInstance(std::shared_ptr<State> s) : state(std::move(s)) {}
std::vector<DynamicNodeInvocation> const &ComputationGraphInstance::get_execution_order() const { return state->order; }
Allocator &ComputationGraphInstance::get_allocator() const { return state->allocator; }
OptimizerAttrs const &ComputationGraphInstance::get_optimizer_attrs() const { return state->optimizer_attrs; }
void ComputationGraphInstance::update_optimizer_attrs_for_next_iter() {
  state->optimizer_attrs = get_optimizer_attrs_for_next_iter(state->optimizer_attrs);
  state->iteration++;
}
std::optional<GenericTensorAccessorR> ComputationGraphInstance::get_loss_tensor_accessor() const {
  if (!state->logit.has_value()) return std::nullopt;
  return read_only_accessor_from_write_accessor(state->grad.at(state->logit->raw).value());
}
GenericTensorAccessorW ComputationGraphInstance::get_tensor_accessor(tensor_guid_t t) const {
  return state->value.at(t.raw);
}
std::optional<GenericTensorAccessorW> ComputationGraphInstance::get_gradient_accessor(tensor_guid_t t) const {
  return state->grad.at(t.raw);
}
std::optional<GenericTensorAccessorW> ComputationGraphInstance::get_master_weight_accessor(tensor_guid_t t) const {
  return state->master.at(t.raw);
}
size_t ComputationGraphInstance::bytes_allocated() const { return state->arena_bytes; }

void ComputationGraphInstance::sync_master_weights() const {
  ffk_stream_t st = get_gpu_device_stream().require_gpu();
  for (size_t t = 0; t < state->master.size(); t++) {
    if (!state->master[t].has_value()) continue;
    GenericTensorAccessorW const &w = state->value[t];
    check_ffk(ffk_cast_forward(st, dt(w.shape.data_type), FFK_FLOAT, w.ptr, state->master[t]->ptr,
                               get_num_elements(w.shape.dims)),
              "sync_master_weights");
  }
  state->masters_valid = true;
}

void ComputationGraphInstance::clear_accumulated_gradients(device_stream_t const &stream) const {
  if (state->cleared_bytes > 0) {
    check_ffk(ffk_fill_zero(state->arena, state->cleared_bytes, stream.require_gpu()), "clear gradients");
  }
}

// ---- planning -------------------------------------------------------------------

namespace {

// how each operator's backward treats the gradients it produces
struct BackwardPlan {
  bool has_backward = false;
  bool accumulate = false;                 // one switch for all input gradients of the op
  std::vector<bool> accumulate_input;      // Linear only: input, weight, bias
  bool softmax_via_scratch = false;
  bool add_by_alias = false;               // ElementBinary add: see alias_of below
};

struct Slot {
  size_t offset = 0, bytes = 0;
};

struct Planner {
  size_t total = 0;
  Slot take(size_t bytes) {
    Slot s{total, bytes};
    total += align_up(bytes);
    return s;
  }
};

struct LayerPlan {
  BackwardPlan bwd;
  Slot saved;        // state kept from forward to backward (LayerNorm statistics, attention reserve)
  size_t scratch_bytes = 0;  // backward scratch, shared between layers ...
  bool own_scratch = false;  // ... unless its partial sums must survive until the end of the pass
  Slot scratch;
};

bool is_op_layer(ComputationGraph::Layer const &l) {
  return !std::holds_alternative<InputAttrs>(l.attrs.op_attrs) && !std::holds_alternative<WeightAttrs>(l.attrs.op_attrs);
}

ffk_mha_desc_t mha_desc(MultiHeadAttentionAttrs const &a, TensorShape const &q, TensorShape const &k, TensorShape const &v) {
  ffk_mha_desc_t d{};
  d.num_samples = dim_at_idx(q.dims, 0);
  d.num_heads = a.num_heads;
  d.q_size = dim_at_idx(q.dims, -1);
  d.k_size = dim_at_idx(k.dims, -1);
  d.v_size = dim_at_idx(v.dims, -1);
  d.q_proj_size = a.kdim;
  d.k_proj_size = a.kdim;
  d.v_proj_size = a.vdim;
  d.o_proj_size = a.embed_dim;
  d.qo_seq_length = dim_at_idx(q.dims, 1);
  d.kv_seq_length = dim_at_idx(k.dims, 1);
  d.scale = a.scale;
  d.causal = a.causal ? 1 : 0;
  return d;
}

int activation_code(std::optional<Activation> const &a) { return a.has_value() ? static_cast<int>(*a) : FFK_ACT_NONE; }

int aggr_code(std::optional<AggregateOp> const &a) {
  if (!a.has_value()) return FFK_AGGR_NONE;
  return *a == AggregateOp::SUM ? FFK_AGGR_SUM : FFK_AGGR_AVG;
}

}  // namespace

ComputationGraphInstance create_computation_graph_instance(
    ComputationGraph const &cg, OptimizerAttrs const &optimizer_attrs, std::optional<LossConfig> const &loss,
    std::unordered_map<tensor_guid_t, GenericTensorAccessorW> const &input_tensors, Allocator &allocator,
    ProfilingSettings const &, device_handle_t const &device_handle, device_id_t device_idx) {
  if (device_idx.device_type != DeviceType::GPU || !device_handle.is_for_gpu() ||
      allocator.get_allocation_device_type() != DeviceType::GPU) {
    bad("NOT_IMPLEMENTED for the CPU device type in this library");
  }
  auto st = std::make_shared<ComputationGraphInstance::State>(cg, allocator, optimizer_attrs);
  size_t const T = cg.tensors.size(), L = cg.layers.size();
  auto shape_of = [&](tensor_guid_t t) -> TensorShape const & { return cg.tensors.at(t.raw).shape; };
  auto numel = [&](tensor_guid_t t) { return get_num_elements(shape_of(t).dims); };

  // -- which tensors carry a gradient, and who writes it
  std::vector<bool> has_grad(T, false), is_weight(T, false);
  for (size_t t = 0; t < T; t++) {
    ComputationGraph::Layer const &src = cg.layers.at(cg.tensors[t].source.raw);
    bool const input_without_grad = std::holds_alternative<InputAttrs>(src.attrs.op_attrs) && cg.tensors[t].create_grad == CreateGrad::NO;
    has_grad[t] = is_float_type(cg.tensors[t].shape.data_type) && !input_without_grad;
    is_weight[t] = std::holds_alternative<WeightAttrs>(src.attrs.op_attrs);
  }
  if (loss.has_value()) {
    st->logit = loss->logit_tensor;
    if (!has_grad.at(loss->logit_tensor.raw)) bad("the logit tensor carries no gradient");
    if (shape_of(loss->logit_tensor).data_type != DataType::FLOAT) bad("the loss kernels take FLOAT logits (cast first)");
  }
  std::vector<int> writers(T, 0);
  for (size_t l = 0; l < L; l++) {
    ComputationGraph::Layer const &layer = cg.layers[l];
    if (!is_op_layer(layer)) continue;
    bool const self_attention = std::holds_alternative<MultiHeadAttentionAttrs>(layer.attrs.op_attrs) &&
                                layer.inputs[0] == layer.inputs[1] && layer.inputs[0] == layer.inputs[2];
    for (size_t i = 0; i < layer.inputs.size(); i++) {
      if (self_attention && i > 0) break;  // key and value gradients are folded into the query's
      if (has_grad[layer.inputs[i].raw]) writers[layer.inputs[i].raw]++;
    }
    for (tensor_guid_t w : layer.weights) writers[w.raw]++;
  }
  auto must_accumulate = [&](tensor_guid_t t) {
    return writers[t.raw] > 1 || (st->logit.has_value() && *st->logit == t);
  };

  // A gradient several operators add into needs no clearing if the one that runs first in the
  // backward pass (the consumer with the highest layer index) stores instead of adding.  That is
  // done where an operator has a switch for this gradient alone: operators with one
  // differentiable input, Linear, and the add whose backward is a copy.
  std::vector<int> first_writer(T, -1);
  std::vector<bool> first_writer_stores(T, false);
  for (size_t l = 0; l < L; l++) {
    ComputationGraph::Layer const &layer = cg.layers[l];
    if (!is_op_layer(layer) || !has_grad[layer.outputs.at(0).raw]) continue;
    for (tensor_guid_t t : layer.inputs) {
      if (has_grad[t.raw]) first_writer[t.raw] = (int)l;
    }
  }
  for (size_t t = 0; t < T; t++) {
    if (first_writer[t] < 0 || writers[t] < 2 || is_weight[t] || (st->logit.has_value() && st->logit->raw == (int)t)) continue;
    ComputationGraph::Layer const &layer = cg.layers[(size_t)first_writer[t]];
    ComputationGraphOpAttrs const &oa = layer.attrs.op_attrs;
    int times = 0;
    for (tensor_guid_t in : layer.inputs) times += in.raw == (int)t;
    bool const one_input = std::holds_alternative<LayerNormAttrs>(oa) || std::holds_alternative<DropoutAttrs>(oa) ||
                           std::holds_alternative<ElementUnaryAttrs>(oa) || std::holds_alternative<TransposeAttrs>(oa) ||
                           std::holds_alternative<ReshapeAttrs>(oa);
    bool const linear_input = std::holds_alternative<LinearAttrs>(oa);
    auto const *bin = std::get_if<ElementBinaryAttrs>(&oa);
    bool const add = bin != nullptr && bin->type == OperatorType::EW_ADD;  // confirmed below, where the add is planned
    first_writer_stores[t] = times == 1 && (one_input || linear_input || add);
  }
  auto adds_here = [&](tensor_guid_t t, size_t l) {
    return must_accumulate(t) && !(first_writer_stores[t.raw] && first_writer[t.raw] == (int)l);
  };

  // -- per-layer backward mode, saved state and scratch
  std::vector<LayerPlan> plan(L);
  std::vector<bool> cleared(T, false);  // gradient must be zero before the backward pass
  // The backward of y = a + b hands dy to both operands.  An operand whose gradient has no
  // other producer does not get a copy: its gradient IS y's gradient memory (complete by the
  // time the add's backward runs, since every consumer of y ran before it, and not written
  // afterwards).  alias_of[a] = y records that; an operand several producers add into gets
  // grad += dy, an operand without a gradient nothing.
  std::vector<int> alias_of(T, -1);
  Planner saved_planner;
  size_t scratch_bytes = 0, discard_bytes = 0;
  for (size_t l = 0; l < L; l++) {
    ComputationGraph::Layer const &layer = cg.layers[l];
    if (!is_op_layer(layer)) continue;
    LayerPlan &p = plan[l];
    ComputationGraphOpAttrs const &oa = layer.attrs.op_attrs;
    bool any_grad = false;
    for (tensor_guid_t t : layer.inputs) any_grad = any_grad || has_grad[t.raw];
    for (tensor_guid_t t : layer.weights) any_grad = any_grad || has_grad[t.raw];
    p.bwd.has_backward = any_grad && has_grad[layer.outputs.at(0).raw];
    bool acc = false;
    for (tensor_guid_t t : layer.inputs) acc = acc || (has_grad[t.raw] && adds_here(t, l));
    if (auto const *a = std::get_if<LinearAttrs>(&oa)) {
      int64_t batch = numel(layer.inputs[0]) / dim_at_idx(shape_of(layer.inputs[0]).dims, -1);
      p.scratch_bytes = ffk_linear_backward_workspace_bytes(dt(shape_of(layer.outputs[0]).data_type), activation_code(a->activation),
                                                            a->use_bias, batch, a->out_channels);
      // one flag per gradient: input, weight, bias (a weight shared between layers is added into)
      p.own_scratch = a->use_bias;  // the bias gradient's last step is collected (ffk_column_reductions_begin)
      p.bwd.accumulate_input = {acc};
      for (tensor_guid_t w : layer.weights) p.bwd.accumulate_input.push_back(writers[w.raw] > 1);
      acc = false;
      if (p.bwd.accumulate_input[0]) cleared[layer.inputs[0].raw] = true;
      for (size_t i = 0; i < layer.weights.size(); i++) {
        if (p.bwd.accumulate_input[1 + i]) cleared[layer.weights[i].raw] = true;
      }
    } else if (std::get_if<LayerNormAttrs>(&oa)) {
      int64_t N = layer.weights.empty() ? 0 : numel(layer.weights[0]);
      auto const *a = std::get_if<LayerNormAttrs>(&oa);
      if (N == 0) {
        N = 1;
        int nd = get_num_dims(shape_of(layer.inputs[0]).dims);
        for (size_t i = 0; i < a->axes.size(); i++) N *= shape_of(layer.inputs[0]).dims.ff_ordered[nd - 1 - (int)i];
      }
      int64_t M = numel(layer.inputs[0]) / N;
      for (tensor_guid_t w : layer.weights) {
        if (writers[w.raw] > 1) bad("LayerNorm weights cannot be shared between layers (their gradients are overwritten)");
      }
      p.saved = saved_planner.take(align_up((size_t)M * 4) * 2);
      p.scratch_bytes = ffk_layer_norm_backward_workspace_bytes(M, N);
      p.own_scratch = !layer.weights.empty();
    } else if (auto const *a = std::get_if<MultiHeadAttentionAttrs>(&oa)) {
      ffk_mha_desc_t d = mha_desc(*a, shape_of(layer.inputs[0]), shape_of(layer.inputs[1]), shape_of(layer.inputs[2]));
      p.saved = saved_planner.take(ffk_mha_reserve_bytes(&d, dt(shape_of(layer.inputs[0]).data_type)));
      // key == value but not the query: both gradients land in one tensor
      if (layer.inputs[1] == layer.inputs[2] && layer.inputs[0] != layer.inputs[1]) acc = true;
      if (layer.inputs[0] == layer.inputs[1] && layer.inputs[0] != layer.inputs[2]) acc = true;
      if (layer.inputs[0] == layer.inputs[2] && layer.inputs[0] != layer.inputs[1]) acc = true;
      // a weight used by one layer has its gradient stored; a shared one is added into
      if (writers[layer.weights.at(0).raw] > 1) cleared[layer.weights.at(0).raw] = true;
    } else if (auto const *a = std::get_if<EmbeddingAttrs>(&oa)) {
      p.scratch_bytes = ffk_embedding_backward_workspace_bytes(numel(layer.inputs[0]), a->num_entries);
      cleared[layer.weights.at(0).raw] = true;
    } else if (std::get_if<SoftmaxAttrs>(&oa)) {
      // the kernel overwrites; with other producers it goes through scratch and is added
      if (acc) {
        p.bwd.softmax_via_scratch = true;
        p.scratch_bytes = (size_t)get_size_in_bytes(shape_of(layer.inputs[0]));
      }
    } else if (std::get_if<ConcatAttrs>(&oa)) {
      // one switch for all parts; the same tensor twice among the inputs is added into
      for (size_t i = 0; i < layer.inputs.size(); i++) {
        for (size_t j = i + 1; j < layer.inputs.size(); j++) acc = acc || layer.inputs[i] == layer.inputs[j];
      }
      if (p.bwd.has_backward && acc && shape_of(layer.outputs[0]).data_type != DataType::FLOAT &&
          shape_of(layer.outputs[0]).data_type != DataType::BF16) {
        bad("concat backward adds in FLOAT or BF16 only");
      }
    } else if (std::get_if<GatherAttrs>(&oa)) {
      // the scatter adds (atomics) into the values' gradient; the index carries none
      if (has_grad[layer.inputs[0].raw]) {
        if (shape_of(layer.inputs[0]).data_type != DataType::FLOAT) bad("gather backward adds FLOAT gradients");
        cleared[layer.inputs[0].raw] = true;
      }
      acc = false;
    } else if (std::get_if<TransposeAttrs>(&oa) || std::get_if<ReshapeAttrs>(&oa)) {
      if (acc && shape_of(layer.outputs[0]).data_type != DataType::FLOAT && shape_of(layer.outputs[0]).data_type != DataType::BF16) {
        bad("transpose / reshape backward adds in FLOAT or BF16 only");
      }
    } else if (std::get_if<CastAttrs>(&oa)) {
      acc = true;  // cast_backward always adds
    } else if (auto const *a = std::get_if<ElementBinaryAttrs>(&oa)) {
      if (p.bwd.has_backward && numel(layer.inputs[0]) != numel(layer.inputs[1])) {
        bad("element binary backward needs operands of equal size");
      }
      if (layer.inputs[0] == layer.inputs[1]) acc = true;
      tensor_guid_t const out = layer.outputs[0];
      if (a->type == OperatorType::EW_ADD && p.bwd.has_backward && layer.inputs[0] != layer.inputs[1]) {
        int cheaper = 0;  // operands that get no kernel (alias) or a copy that saves a clearing fill
        bool all_handled = true;
        for (tensor_guid_t t : layer.inputs) {
          bool const same = shape_of(t) == shape_of(out);
          if (!has_grad[t.raw]) continue;
          if (same && !must_accumulate(t) && !is_weight[t.raw]) cheaper++;
          else if (same && must_accumulate(t)) cheaper += !adds_here(t, l);
          else all_handled = false;
        }
        if (all_handled && cheaper > 0) {
          p.bwd.add_by_alias = true;
          acc = false;
          for (tensor_guid_t t : layer.inputs) {
            if (!has_grad[t.raw]) continue;
            if (!must_accumulate(t)) alias_of[t.raw] = out.raw;
            else if (adds_here(t, l)) cleared[t.raw] = true;
          }
        } else {
          for (tensor_guid_t t : layer.inputs) {
            if (first_writer[t.raw] == (int)l) first_writer_stores[t.raw] = false;  // the plain kernel adds
          }
          acc = false;
          for (tensor_guid_t t : layer.inputs) acc = acc || (has_grad[t.raw] && adds_here(t, l));
          if (layer.inputs[0] == layer.inputs[1]) acc = true;
        }
      } else {
        for (tensor_guid_t t : layer.inputs) {
          if (first_writer[t.raw] == (int)l) first_writer_stores[t.raw] = false;  // not an add after all
        }
        acc = false;
        for (tensor_guid_t t : layer.inputs) acc = acc || (has_grad[t.raw] && adds_here(t, l));
        if (layer.inputs[0] == layer.inputs[1]) acc = true;
      }
    }
    p.bwd.accumulate = acc;
    if (acc) {
      for (tensor_guid_t t : layer.inputs) {
        if (has_grad[t.raw]) cleared[t.raw] = true;
      }
    }
    if (!p.own_scratch) scratch_bytes = std::max(scratch_bytes, p.scratch_bytes);
    // an input without a gradient still needs somewhere for the kernel to write
    if (p.bwd.has_backward && !std::holds_alternative<LinearAttrs>(oa) && !std::holds_alternative<EmbeddingAttrs>(oa)) {
      for (tensor_guid_t t : layer.inputs) {
        if (!has_grad[t.raw]) discard_bytes = std::max(discard_bytes, (size_t)get_size_in_bytes(shape_of(t)));
      }
    }
  }
  if (st->logit.has_value()) cleared[st->logit->raw] = false;  // written by the loss before any producer adds
  for (size_t t = 0; t < T; t++) {
    if (first_writer_stores[t]) cleared[t] = false;  // its first producer stores
  }

  // -- neighbouring operators run as one kernel where the library has one that produces the
  // same bits (ffk_set_option(FFK_OPTION_LAYER_UNFUSED, 1) switches this off).  The intermediate tensor of a fused pair
  // has that pair's second operator as its only consumer and is never written.
  //   GELU -> Dropout:            forward one kernel at the Dropout, backward one at the GELU
  //   Dropout -> element-wise add: forward one kernel at the add (the backward of the add copies
  //                                nothing, see alias_of, and the Dropout's is its own)
  enum class Fused { NONE, GELU_DROPOUT_HEAD, GELU_DROPOUT_TAIL, DROPOUT_ADD_HEAD, DROPOUT_ADD_TAIL };
  std::vector<Fused> fused(L, Fused::NONE);
  std::vector<size_t> partner(L, 0);
  // A Linear next to a fused pair takes the pair onto its GEMM's tile store (BF16 shapes the
  // library has such a kernel for; for the others the Linear's invocation runs the two launches):
  //   Linear -> (Dropout -> add):   linear_sum[linear] = the add, sum_linear[add] = the Linear;
  //                                 the Linear's forward writes the add's output
  //   (GELU -> Dropout) -> Linear:  linear_gelu[linear] = the GELU, gelu_linear[gelu] = the Linear;
  //                                 the Linear's backward writes the gradient of the GELU's input
  std::vector<int> linear_sum(L, -1), sum_linear(L, -1), linear_gelu(L, -1), gelu_linear(L, -1);
  // A LayerNorm next to the residual add of its block:
  //   ln_residual[ln] = the add (a LATER layer) that reads the LayerNorm's input t as an operand.  Going back, that
  //     add runs first and would copy its output gradient into t's; instead the LayerNorm's backward reads that
  //     output gradient as a residual and writes t's gradient whole (deferred_to_ln[t] = ln: the add skips t).
  //   ln_drop[ln] = the Dropout whose output was the other operand of the add that PRODUCED t: t's gradient is
  //     complete once the LayerNorm (its last producer) has run, and the same kernel writes the gradient of
  //     the Dropout's input (drop_bwd_by_ln[dropout]: its own backward does nothing).
  //   ln_pre[ln] = that producing add, when it and its Dropout are a fused pair no Linear has taken: the
  //     LayerNorm's forward computes the sum as well (add_fwd_by_ln[add]: its own forward does nothing).
  std::vector<int> ln_residual(L, -1), ln_drop(L, -1), ln_pre(L, -1), deferred_to_ln(T, -1);
  std::vector<bool> drop_bwd_by_ln(L, false), add_fwd_by_ln(L, false);
  // The bias gradient of a Linear (the column sums of its output's gradient) taken by the kernel that
  // produces that gradient:
  //   drop_bias[dropout] = the Linear whose output the Dropout reads: the Dropout's backward sums as it writes;
  //   gelu_bias[linear]  = the Linear whose output the GELU of a (GELU -> Dropout) -> Linear chain reads: the
  //                        second Linear's input-gradient GEMM sums on its tile store.
  // Whether the library had such a kernel for the shape is only known when the call returns, so the producer
  // leaves word for the Linear (bias_done[linear], written and read once per step, in that order).
  std::vector<int> drop_bias(L, -1), gelu_bias(L, -1);
  std::vector<std::shared_ptr<bool>> bias_done(L);
  {
    int unfused = 0;
    check_ffk(ffk_get_option(FFK_OPTION_LAYER_UNFUSED, &unfused), "ffk_get_option");
    bool const enabled = unfused == 0;
    std::vector<int> uses(T, 0);
    std::vector<size_t> consumer(T, 0);
    for (size_t l = 0; l < L; l++) {
      if (!is_op_layer(cg.layers[l])) continue;
      for (tensor_guid_t t : cg.layers[l].inputs) uses[t.raw]++, consumer[t.raw] = l;
    }
    auto vectorizable = [&](tensor_guid_t t) {
      DataType const d = shape_of(t).data_type;
      return (d == DataType::FLOAT || d == DataType::BF16) && numel(t) % 8 == 0;
    };
    // what the instance places is 256-byte aligned; caller memory has to be looked at
    auto aligned = [&](tensor_guid_t t) {
      auto bound = input_tensors.find(t);
      return bound == input_tensors.end() || reinterpret_cast<uintptr_t>(bound->second.ptr) % 16 == 0;
    };
    auto only_consumer = [&](tensor_guid_t t, size_t &c) {
      if (uses[t.raw] != 1 || (st->logit.has_value() && *st->logit == t)) return false;
      c = consumer[t.raw];
      return fused[c] == Fused::NONE;
    };
    for (size_t l = 0; enabled && l < L; l++) {
      ComputationGraph::Layer const &layer = cg.layers[l];
      if (!is_op_layer(layer) || fused[l] != Fused::NONE) continue;
      tensor_guid_t const out = layer.outputs.at(0);
      size_t c = 0;
      if (auto const *u = std::get_if<ElementUnaryAttrs>(&layer.attrs.op_attrs)) {
        if (u->op_type != OperatorType::GELU || !vectorizable(out) || !only_consumer(out, c)) continue;
        if (!std::holds_alternative<DropoutAttrs>(cg.layers[c].attrs.op_attrs)) continue;
        bool const any_bwd = plan[l].bwd.has_backward || plan[c].bwd.has_backward;
        bool const both_bwd = plan[l].bwd.has_backward && plan[c].bwd.has_backward && !plan[l].bwd.accumulate &&
                              has_grad[layer.inputs[0].raw];
        if (any_bwd && !both_bwd) continue;
        if (!aligned(layer.inputs[0]) || !aligned(cg.layers[c].outputs.at(0))) continue;
        fused[l] = Fused::GELU_DROPOUT_HEAD, fused[c] = Fused::GELU_DROPOUT_TAIL, partner[l] = c, partner[c] = l;
      } else if (std::holds_alternative<DropoutAttrs>(layer.attrs.op_attrs)) {
        if (!vectorizable(out) || !only_consumer(out, c)) continue;
        auto const *b = std::get_if<ElementBinaryAttrs>(&cg.layers[c].attrs.op_attrs);
        if (b == nullptr || b->type != OperatorType::EW_ADD) continue;
        ComputationGraph::Layer const &add = cg.layers[c];
        tensor_guid_t const other = add.inputs[0] == out ? add.inputs[1] : add.inputs[0];
        if (other == out || !(shape_of(other) == shape_of(out))) continue;
        if (!aligned(layer.inputs[0]) || !aligned(other) || !aligned(add.outputs.at(0))) continue;
        fused[l] = Fused::DROPOUT_ADD_HEAD, fused[c] = Fused::DROPOUT_ADD_TAIL, partner[l] = c, partner[c] = l;
      }
    }
    std::vector<int> producer(T, -1);  // the operator layer a tensor comes from (-1: an input or a weight)
    for (size_t l = 0; l < L; l++) {
      if (!is_op_layer(cg.layers[l])) continue;
      for (tensor_guid_t t : cg.layers[l].outputs) producer[t.raw] = (int)l;
    }
    auto plain_bf16_linear = [&](int l) {
      if (l < 0) return false;
      auto const *a = std::get_if<LinearAttrs>(&cg.layers[l].attrs.op_attrs);
      return a != nullptr && !a->activation.has_value() &&
             shape_of(cg.layers[l].outputs.at(0)).data_type == DataType::BF16 && aligned(cg.layers[l].inputs[0]);
    };
    auto single_use = [&](tensor_guid_t t) { return uses[t.raw] == 1 && !(st->logit.has_value() && *st->logit == t); };
    for (size_t l = 0; enabled && l < L; l++) {
      if (fused[l] == Fused::DROPOUT_ADD_HEAD) {
        ComputationGraph::Layer const &drop = cg.layers[l], &add = cg.layers[partner[l]];
        int const lin = producer[drop.inputs[0].raw];
        if (!plain_bf16_linear(lin) || !single_use(drop.inputs[0])) continue;
        tensor_guid_t const other = add.inputs[0] == drop.outputs.at(0) ? add.inputs[1] : add.inputs[0];
        if (producer[other.raw] >= lin) continue;  // the other operand must exist when the Linear runs
        linear_sum[lin] = (int)partner[l], sum_linear[partner[l]] = lin;
      } else if (fused[l] == Fused::GELU_DROPOUT_HEAD && plan[l].bwd.has_backward) {
        tensor_guid_t const dropped = cg.layers[partner[l]].outputs.at(0);
        if (!single_use(dropped)) continue;
        int const lin = (int)consumer[dropped.raw];
        if (!plain_bf16_linear(lin) || cg.layers[lin].inputs[0] != dropped) continue;
        if (!plan[lin].bwd.has_backward || plan[lin].bwd.accumulate_input[0]) continue;
        linear_gelu[lin] = (int)l, gelu_linear[l] = lin;
      }
    }
    std::vector<int> first_consumer(T, -1);
    for (size_t l = L; l-- > 0;) {
      if (!is_op_layer(cg.layers[l])) continue;
      for (tensor_guid_t t : cg.layers[l].inputs) first_consumer[t.raw] = (int)l;
    }
    for (size_t n = 0; enabled && n < L; n++) {
      ComputationGraph::Layer const &ln = cg.layers[n];
      if (!is_op_layer(ln) || !std::holds_alternative<LayerNormAttrs>(ln.attrs.op_attrs)) continue;
      tensor_guid_t const t = ln.inputs[0];
      DataType const type = shape_of(t).data_type;
      if ((type != DataType::FLOAT && type != DataType::BF16) || !aligned(t) || !aligned(ln.outputs.at(0))) continue;
      int const made_by = producer[t.raw];
      bool const made_by_pair = made_by >= 0 && fused[made_by] == Fused::DROPOUT_ADD_TAIL;
      // forward: Dropout -> add -> this LayerNorm, the LayerNorm being the sum's first reader
      if (made_by_pair && sum_linear[made_by] < 0 && type == DataType::BF16 && first_consumer[t.raw] == (int)n) {
        ln_pre[n] = made_by;
        add_fwd_by_ln[made_by] = true;
      }
      // backward: the later add's copy into t's gradient becomes this LayerNorm's residual
      if (!plan[n].bwd.has_backward || !has_grad[t.raw] || writers[t.raw] != 2 || is_weight[t.raw]) continue;
      if (st->logit.has_value() && *st->logit == t) continue;
      int const l = first_writer[t.raw];
      if (l <= (int)n || !first_writer_stores[t.raw] || alias_of[t.raw] >= 0) continue;
      auto const *b = std::get_if<ElementBinaryAttrs>(&cg.layers[l].attrs.op_attrs);
      if (b == nullptr || b->type != OperatorType::EW_ADD || !plan[l].bwd.add_by_alias) continue;
      if (!(shape_of(cg.layers[l].outputs.at(0)) == shape_of(t))) continue;
      ln_residual[n] = l;
      deferred_to_ln[t.raw] = (int)n;
      // ... and with t's gradient complete here, the backward of the Dropout that fed the producing add
      if (!made_by_pair || type != DataType::BF16) continue;
      size_t const d = partner[made_by];
      tensor_guid_t const dropped = cg.layers[d].outputs.at(0), drop_in = cg.layers[d].inputs[0];
      if (alias_of[dropped.raw] != t.raw || !plan[d].bwd.has_backward || plan[d].bwd.accumulate) continue;
      if (!has_grad[drop_in.raw] || writers[drop_in.raw] != 1 || !aligned(drop_in)) continue;
      ln_drop[n] = (int)d;
      drop_bwd_by_ln[d] = true;
    }
    auto biased_plain_linear = [&](int lin, tensor_guid_t out) {
      if (lin < 0) return false;
      auto const *a = std::get_if<LinearAttrs>(&cg.layers[lin].attrs.op_attrs);
      if (a == nullptr || !a->use_bias || a->activation.has_value() || !single_use(out)) return false;
      DataType const type = shape_of(out).data_type;
      return (type == DataType::FLOAT || type == DataType::BF16) && plan[lin].bwd.has_backward &&
             has_grad[cg.layers[lin].weights.at(1).raw] && has_grad[out.raw];
    };
    for (size_t l = 0; enabled && l < L; l++) {
      ComputationGraph::Layer const &layer = cg.layers[l];
      if (!is_op_layer(layer)) continue;
      if (std::holds_alternative<DropoutAttrs>(layer.attrs.op_attrs)) {
        if (drop_bwd_by_ln[l] || fused[l] == Fused::GELU_DROPOUT_TAIL) continue;  // its backward runs elsewhere
        if (!plan[l].bwd.has_backward || plan[l].bwd.accumulate) continue;
        int const lin = producer[layer.inputs[0].raw];
        if (!biased_plain_linear(lin, layer.inputs[0])) continue;
        drop_bias[l] = lin;
        bias_done[lin] = std::make_shared<bool>(false);
      } else if (linear_gelu[l] >= 0) {
        tensor_guid_t const u = cg.layers[(size_t)linear_gelu[l]].inputs[0];
        int const lin = producer[u.raw];
        if (!biased_plain_linear(lin, u) || shape_of(u).data_type != DataType::BF16) continue;
        gelu_bias[l] = lin;
        bias_done[lin] = std::make_shared<bool>(false);
      }
    }
  }

  // -- placement: cleared gradients first, then everything else.
  // Trainable weights that the instance places itself are laid out in groups
  // (same data type, gradient cleared or not): within a group the gradient, the
  // value, the fp32 master and the optimizer moments of all members lie in
  // parallel arrays at the same element offsets (members padded to 128
  // elements), so that ONE update launch over the group's extent updates every
  // member; the padding is updated too and never read.
  Planner arena;
  std::vector<Slot> grad_slot(T), value_slot(T), master_slot(T), v_slot(T), m_slot(T);
  bool const adam = std::holds_alternative<AdamOptimizerAttrs>(optimizer_attrs);
  bool const sgd_momentum = !adam && std::get<SGDOptimizerAttrs>(optimizer_attrs).momentum > 0.0;
  struct WeightGroup {
    DataType type;
    bool cleared;
    std::vector<size_t> members;
    std::vector<size_t> elem_offset;
    size_t elems = 0;
    Slot grad, value, master, v, m;
  };
  std::vector<WeightGroup> groups;
  std::vector<int> group_of(T, -1);
  for (size_t t = 0; t < T; t++) {
    if (!is_weight[t] || !has_grad[t]) continue;
    TensorShape const &s = cg.tensors[t].shape;
    if (s.data_type != DataType::FLOAT && s.data_type != DataType::BF16) bad("weights must be FLOAT or BF16");
    if (input_tensors.count(tensor_guid_t{(int)t}) != 0) continue;  // lives in the caller's memory: updated on its own
    size_t g = 0;
    while (g < groups.size() && !(groups[g].type == s.data_type && groups[g].cleared == cleared[t])) g++;
    if (g == groups.size()) groups.push_back(WeightGroup{s.data_type, cleared[t], {}, {}, 0, {}, {}, {}, {}, {}});
    group_of[t] = (int)g;
    groups[g].members.push_back(t);
    groups[g].elem_offset.push_back(groups[g].elems);
    groups[g].elems += ((size_t)get_num_elements(s.dims) + 127) & ~(size_t)127;
  }
  auto place_group_gradients = [&](bool cleared_ones) {
    for (WeightGroup &g : groups) {
      if (g.cleared != cleared_ones) continue;
      size_t const es = (size_t)size_of_datatype(g.type);
      g.grad = arena.take(g.elems * es);
      for (size_t i = 0; i < g.members.size(); i++) {
        size_t const t = g.members[i];
        grad_slot[t] = Slot{g.grad.offset + g.elem_offset[i] * es, (size_t)get_size_in_bytes(cg.tensors[t].shape)};
      }
    }
  };
  place_group_gradients(true);
  for (size_t t = 0; t < T; t++) {
    if (has_grad[t] && cleared[t] && group_of[t] < 0) grad_slot[t] = arena.take((size_t)get_size_in_bytes(cg.tensors[t].shape));
  }
  st->cleared_bytes = arena.total;
  place_group_gradients(false);
  for (WeightGroup &g : groups) {
    size_t const es = (size_t)size_of_datatype(g.type);
    g.value = arena.take(g.elems * es);
    if (g.type == DataType::BF16) g.master = arena.take(g.elems * 4);
    if (adam || sgd_momentum) g.v = arena.take(g.elems * 4);
    if (adam) g.m = arena.take(g.elems * 4);
    for (size_t i = 0; i < g.members.size(); i++) {
      size_t const t = g.members[i], n = (size_t)get_num_elements(cg.tensors[t].shape.dims), eo = g.elem_offset[i];
      value_slot[t] = Slot{g.value.offset + eo * es, n * es};
      if (g.master.bytes) master_slot[t] = Slot{g.master.offset + eo * 4, n * 4};
      if (g.v.bytes) v_slot[t] = Slot{g.v.offset + eo * 4, n * 4};
      if (g.m.bytes) m_slot[t] = Slot{g.m.offset + eo * 4, n * 4};
    }
  }
  for (size_t t = 0; t < T; t++) {
    if (group_of[t] >= 0) continue;
    TensorShape const &s = cg.tensors[t].shape;
    if (has_grad[t] && !cleared[t] && alias_of[t] < 0) grad_slot[t] = arena.take((size_t)get_size_in_bytes(s));
    if (input_tensors.count(tensor_guid_t{(int)t}) == 0) value_slot[t] = arena.take((size_t)get_size_in_bytes(s));
    if (is_weight[t] && has_grad[t]) {
      size_t f32 = (size_t)get_num_elements(s.dims) * 4;
      if (s.data_type == DataType::BF16) master_slot[t] = arena.take(f32);
      if (adam || sgd_momentum) v_slot[t] = arena.take(f32);
      if (adam) m_slot[t] = arena.take(f32);
    }
  }
  for (size_t t = 0; t < T; t++) {
    if (alias_of[t] < 0) continue;
    int root = alias_of[t];
    while (alias_of[(size_t)root] >= 0) root = alias_of[(size_t)root];
    grad_slot[t] = grad_slot[(size_t)root];
  }
  size_t const saved_base = arena.take(saved_planner.total).offset;
  size_t const scratch_base = arena.take(scratch_bytes).offset;
  for (size_t l = 0; l < L; l++) {
    if (plan[l].own_scratch && plan[l].scratch_bytes > 0) plan[l].scratch = arena.take(plan[l].scratch_bytes);
  }
  size_t const discard_base = arena.take(discard_bytes).offset;
  st->arena_bytes = arena.total;
  st->arena = static_cast<char *>(allocator.allocate(std::max<size_t>(arena.total, 256)));
  // optimizer moments start at zero; so do gradients nobody writes
  check_ffk(ffk_fill_zero(st->arena, std::max<size_t>(arena.total, 256), nullptr), "create_computation_graph_instance");
  check_ffk(ffk_stream_synchronize(nullptr), "create_computation_graph_instance");

  char *const base = st->arena;
  auto f32_accessor = [&](size_t t, Slot const &s) -> std::optional<GenericTensorAccessorW> {
    if (s.bytes == 0) return std::nullopt;
    return GenericTensorAccessorW{TensorShape{cg.tensors[t].shape.dims, DataType::FLOAT}, base + s.offset, DeviceType::GPU};
  };
  st->value.resize(T, GenericTensorAccessorW{TensorShape{TensorDims{{}}, DataType::FLOAT}, nullptr, DeviceType::GPU});
  st->grad.resize(T);
  st->master.resize(T);
  st->opt_v.resize(T);
  st->opt_m.resize(T);
  for (size_t t = 0; t < T; t++) {
    auto bound = input_tensors.find(tensor_guid_t{(int)t});
    if (bound != input_tensors.end()) {
      if (bound->second.shape != cg.tensors[t].shape) bad("a bound tensor has the wrong shape");
      if (bound->second.device_type != DeviceType::GPU) bad("a bound tensor is not device-resident");
      st->value[t] = bound->second;
    } else {
      st->value[t] = GenericTensorAccessorW{cg.tensors[t].shape, base + value_slot[t].offset, DeviceType::GPU};
    }
    if (has_grad[t]) st->grad[t] = GenericTensorAccessorW{cg.tensors[t].shape, base + grad_slot[t].offset, DeviceType::GPU};
    st->master[t] = f32_accessor(t, master_slot[t]);
    st->opt_v[t] = f32_accessor(t, v_slot[t]);
    st->opt_m[t] = f32_accessor(t, m_slot[t]);
  }
  void *const shared_scratch = base + scratch_base;
  void *const discard = base + discard_base;
  ComputationGraphInstance::State *const S = st.get();  // closures must not own the state they live in

  auto val = [&](tensor_guid_t t) { return st->value[t.raw].ptr; };
  auto grd = [&](tensor_guid_t t) -> void * { return has_grad[t.raw] ? st->grad[t.raw]->ptr : nullptr; };
  auto grd_or_discard = [&](tensor_guid_t t) -> void * { return has_grad[t.raw] ? st->grad[t.raw]->ptr : discard; };

  // -- FWD / BWD invocations
  std::vector<DynamicNodeInvocation> fwd, bwd;
  for (size_t l = 0; l < L; l++) {
    ComputationGraph::Layer const &layer = cg.layers[l];
    if (!is_op_layer(layer)) continue;
    LayerPlan const &p = plan[l];
    ComputationGraphOpAttrs const &oa = layer.attrs.op_attrs;
    layer_guid_t const id{(int)l};
    tensor_guid_t const out = layer.outputs.at(0);
    void *const y = val(out);
    void *const dy = grd(out);
    size_t const ws_bytes = p.scratch_bytes;
    void *const scratch = p.own_scratch ? static_cast<void *>(base + p.scratch.offset) : shared_scratch;
    std::function<void(device_stream_t const &)> f, b;

    if (auto const *a = std::get_if<LinearAttrs>(&oa)) {
      tensor_guid_t x = layer.inputs[0];
      int const type = dt(shape_of(x).data_type), act = activation_code(a->activation);
      int64_t const in_dim = dim_at_idx(shape_of(x).dims, -1), out_dim = a->out_channels, batch = numel(x) / in_dim;
      void *xp = val(x), *w = val(layer.weights[0]), *bias = a->use_bias ? val(layer.weights[1]) : nullptr;
      void *dx = grd(x), *dw = grd(layer.weights[0]), *dbias = a->use_bias ? grd(layer.weights[1]) : nullptr;
      int const accumulate = (p.bwd.accumulate_input[0] ? FFK_ACC_INPUT : 0) | (p.bwd.accumulate_input[1] ? FFK_ACC_WEIGHT : 0) |
                             (a->use_bias && p.bwd.accumulate_input[2] ? FFK_ACC_BIAS : 0);
      f = [=](device_stream_t const &s) {
        check_ffk(ffk_linear_forward(s.require_gpu(), type, act, xp, y, w, bias, batch, in_dim, out_dim), "Linear forward");
      };
      // the bias gradient, unless the kernel that wrote dy has summed it already this step
      std::shared_ptr<bool> const bias_elsewhere = bias_done[l];
      auto bias_grad_now = [dbias, bias_elsewhere]() -> void * { return bias_elsewhere && *bias_elsewhere ? nullptr : dbias; };
      b = [=](device_stream_t const &s) {
        check_ffk(ffk_linear_backward(s.require_gpu(), type, act, 0, y, dy, xp, dx, w, dw, bias_grad_now(), batch, in_dim, out_dim,
                                      ws_bytes ? scratch : nullptr, ws_bytes, accumulate),
                  "Linear backward");
      };
      if (linear_sum[l] >= 0) {
        // residual + dropout(this Linear), written where the add's output lives
        ComputationGraph::Layer const &add = cg.layers[linear_sum[l]];
        size_t const d = partner[linear_sum[l]];
        ComputationGraph::Layer const &drop = cg.layers[d];
        DropoutAttrs const &da = std::get<DropoutAttrs>(drop.attrs.op_attrs);
        float const rate = da.rate;
        uint64_t const seed = da.seed + (uint64_t)d;
        int64_t const n = numel(out);
        void *residual = val(add.inputs[0] == drop.outputs.at(0) ? add.inputs[1] : add.inputs[0]);
        void *sum = val(add.outputs.at(0));
        f = [=](device_stream_t const &s) {
          uint64_t const offset = S->iteration * (uint64_t)n;
          int const rc = ffk_linear_dropout_add_forward(s.require_gpu(), type, xp, residual, sum, w, bias, batch, in_dim, out_dim,
                                                        rate, seed, offset);
          if (rc != FFK_ERR_UNSUPPORTED) return check_ffk(rc, "Linear + Dropout + add forward");
          check_ffk(ffk_linear_forward(s.require_gpu(), type, act, xp, y, w, bias, batch, in_dim, out_dim), "Linear forward");
          check_ffk(ffk_dropout_add_forward(s.require_gpu(), type, y, residual, sum, n, rate, seed, offset), "Dropout + add forward");
        };
      }
      if (linear_gelu[l] >= 0) {
        // the gradient of this Linear's input goes through the Dropout's and the GELU's backward on its way out
        size_t const g = (size_t)linear_gelu[l], d = partner[g];
        DropoutAttrs const &da = std::get<DropoutAttrs>(cg.layers[d].attrs.op_attrs);
        float const rate = da.rate;
        uint64_t const seed = da.seed + (uint64_t)d;
        int64_t const n = numel(x);
        void *gelu_in = val(cg.layers[g].inputs[0]), *gelu_in_grad = grd(cg.layers[g].inputs[0]);
        int const acc_w = accumulate & ~FFK_ACC_INPUT;
        // the bias gradient of the Linear in front of the GELU, summed where this GEMM stores
        int const first = gelu_bias[l];
        std::shared_ptr<bool> const first_done = first >= 0 ? bias_done[(size_t)first] : nullptr;
        void *first_dbias = first >= 0 ? grd(cg.layers[(size_t)first].weights.at(1)) : nullptr;
        int const first_acc = first >= 0 && plan[(size_t)first].bwd.accumulate_input.at(2) ? 1 : 0;
        void *first_scratch = first >= 0 ? static_cast<void *>(base + plan[(size_t)first].scratch.offset) : nullptr;
        size_t const first_scratch_bytes = first >= 0 ? plan[(size_t)first].scratch_bytes : 0;
        b = [=](device_stream_t const &s) {
          uint64_t const offset = S->iteration * (uint64_t)n;
          void *const bias_grad = bias_grad_now();
          if (first_done) {
            int const rc = ffk_linear_backward_dropout_gelu_bias_grad(
                s.require_gpu(), type, dy, xp, gelu_in, gelu_in_grad, w, dw, bias_grad, batch, in_dim, out_dim,
                ws_bytes ? scratch : nullptr, ws_bytes, acc_w, rate, seed, offset, first_dbias, first_acc, first_scratch,
                first_scratch_bytes);
            *first_done = rc == FFK_OK;
            if (rc != FFK_ERR_UNSUPPORTED) return check_ffk(rc, "Linear + Dropout + GELU backward with bias gradient");
          }
          int const rc = ffk_linear_backward_dropout_gelu(s.require_gpu(), type, dy, xp, gelu_in, gelu_in_grad, w, dw, bias_grad, batch,
                                                          in_dim, out_dim, ws_bytes ? scratch : nullptr, ws_bytes, acc_w, rate, seed,
                                                          offset);
          if (rc != FFK_ERR_UNSUPPORTED) return check_ffk(rc, "Linear + Dropout + GELU backward");
          check_ffk(ffk_linear_backward(s.require_gpu(), type, act, 0, y, dy, xp, dx, w, dw, bias_grad, batch, in_dim, out_dim,
                                        ws_bytes ? scratch : nullptr, ws_bytes, accumulate),
                    "Linear backward");
          check_ffk(ffk_dropout_gelu_backward(s.require_gpu(), type, dx, gelu_in, gelu_in_grad, n, rate, seed, offset),
                    "Dropout + GELU backward");
        };
      }
      if (a->regularizer.has_value()) {
        // the regulariser's term behind the weight-gradient product of every backward call
        // (lib/kernels/src/cuda/ops/linear_kernels.cu:269-290)
        auto const *l2 = std::get_if<L2RegularizerAttrs>(&*a->regularizer);
        if (l2 == nullptr) throw std::runtime_error("Linear: Only L2 regularization is supported");
        float const lambda = l2->lambda;
        int64_t const w_elems = numel(layer.weights[0]);
        int const w_type = dt(shape_of(layer.weights[0]).data_type);
        auto const inner = b;
        b = [=](device_stream_t const &s) {
          inner(s);
          check_ffk(ffk_linear_l2_regularizer_grad(s.require_gpu(), w_type, w, dw, w_elems, lambda), "Linear L2 regularizer");
        };
      }
    } else if (auto const *a = std::get_if<LayerNormAttrs>(&oa)) {
      tensor_guid_t x = layer.inputs[0];
      int const type = dt(shape_of(x).data_type);
      int64_t N = 1;
      int nd = get_num_dims(shape_of(x).dims);
      for (size_t i = 0; i < a->axes.size(); i++) N *= shape_of(x).dims.ff_ordered[nd - 1 - (int)i];
      int64_t const M = numel(x) / N;
      float *mean = reinterpret_cast<float *>(base + saved_base + p.saved.offset);
      float *rstd = reinterpret_cast<float *>(base + saved_base + p.saved.offset + align_up((size_t)M * 4));
      void *xp = val(x), *dx = grd_or_discard(x);
      void *gamma = a->elementwise_affine ? val(layer.weights[0]) : nullptr;
      void *beta = a->elementwise_affine ? val(layer.weights[1]) : nullptr;
      void *dgamma = a->elementwise_affine ? grd(layer.weights[0]) : nullptr;
      void *dbeta = a->elementwise_affine ? grd(layer.weights[1]) : nullptr;
      float const eps = a->eps;
      int const accumulate = p.bwd.accumulate ? 1 : 0;
      f = [=](device_stream_t const &s) {
        check_ffk(ffk_layer_norm_forward(s.require_gpu(), type, xp, y, gamma, beta, mean, rstd, M, N, eps), "LayerNorm forward");
      };
      b = [=](device_stream_t const &s) {
        check_ffk(ffk_layer_norm_backward(s.require_gpu(), type, dy, xp, mean, rstd, gamma, dx, dgamma, dbeta, M, N, scratch,
                                          ws_bytes, accumulate),
                  "LayerNorm backward");
      };
      if (ln_pre[l] >= 0) {
        // x = residual + dropout(u) is computed here, where the add's output lives
        ComputationGraph::Layer const &add = cg.layers[(size_t)ln_pre[l]];
        size_t const d = partner[(size_t)ln_pre[l]];
        ComputationGraph::Layer const &drop = cg.layers[d];
        DropoutAttrs const &da = std::get<DropoutAttrs>(drop.attrs.op_attrs);
        float const rate = da.rate;
        uint64_t const seed = da.seed + (uint64_t)d;
        int64_t const n = numel(x);
        void *u = val(drop.inputs[0]);
        void *residual = val(add.inputs[0] == drop.outputs.at(0) ? add.inputs[1] : add.inputs[0]);
        f = [=](device_stream_t const &s) {
          uint64_t const offset = S->iteration * (uint64_t)n;
          int const rc = ffk_dropout_add_layer_norm_forward(s.require_gpu(), type, u, residual, xp, y, gamma, beta, mean, rstd, M,
                                                            N, eps, rate, seed, offset);
          if (rc != FFK_ERR_UNSUPPORTED) return check_ffk(rc, "Dropout + add + LayerNorm forward");
          check_ffk(ffk_dropout_add_forward(s.require_gpu(), type, u, residual, xp, n, rate, seed, offset), "Dropout + add forward");
          check_ffk(ffk_layer_norm_forward(s.require_gpu(), type, xp, y, gamma, beta, mean, rstd, M, N, eps), "LayerNorm forward");
        };
      }
      if (ln_residual[l] >= 0) {
        void *residual = grd(cg.layers[(size_t)ln_residual[l]].outputs.at(0));
        int64_t const n = numel(x);
        int const acc_params = 0;
        void *dropped_grad = nullptr;
        float rate = 0.0f;
        uint64_t seed = 0;
        if (ln_drop[l] >= 0) {
          size_t const d = (size_t)ln_drop[l];
          DropoutAttrs const &da = std::get<DropoutAttrs>(cg.layers[d].attrs.op_attrs);
          dropped_grad = grd(cg.layers[d].inputs[0]);
          rate = da.rate;
          seed = da.seed + (uint64_t)d;
        }
        b = [=](device_stream_t const &s) {
          uint64_t const offset = S->iteration * (uint64_t)n;
          int const rc = ffk_layer_norm_backward_residual(s.require_gpu(), type, dy, xp, mean, rstd, gamma, residual, dx, dgamma,
                                                          dbeta, M, N, scratch, ws_bytes, acc_params, dropped_grad, rate, seed,
                                                          offset);
          if (rc != FFK_ERR_UNSUPPORTED) return check_ffk(rc, "LayerNorm backward with residual");
          check_ffk(ffk_cast_forward(s.require_gpu(), type, type, residual, dx, n), "ElementBinary backward");
          check_ffk(ffk_layer_norm_backward(s.require_gpu(), type, dy, xp, mean, rstd, gamma, dx, dgamma, dbeta, M, N, scratch,
                                            ws_bytes, FFK_LN_ACC_INPUT),
                    "LayerNorm backward");
          if (dropped_grad != nullptr) {
            check_ffk(ffk_dropout_backward(s.require_gpu(), type, dx, dropped_grad, n, rate, seed, offset, 0), "Dropout backward");
          }
        };
      }
    } else if (auto const *a = std::get_if<MultiHeadAttentionAttrs>(&oa)) {
      tensor_guid_t q = layer.inputs[0], k = layer.inputs[1], v = layer.inputs[2];
      int const type = dt(shape_of(q).data_type);
      ffk_mha_desc_t const d = mha_desc(*a, shape_of(q), shape_of(k), shape_of(v));
      void *reserve = base + saved_base + p.saved.offset;
      size_t const reserve_bytes = p.saved.bytes;
      void *qp = val(q), *kp = val(k), *vp = val(v), *w = val(layer.weights[0]), *dw = grd(layer.weights[0]);
      void *dq = grd_or_discard(q);
      void *dk = k == q ? nullptr : grd_or_discard(k);
      void *dv = v == q ? nullptr : grd_or_discard(v);
      if ((dk == nullptr) != (dv == nullptr)) bad("attention: key and value must both alias the query, or neither");
      int const accumulate = (p.bwd.accumulate ? FFK_MHA_ACC_INPUT_GRADS : 0) |
                             (writers[layer.weights[0].raw] > 1 ? 0 : FFK_MHA_OVERWRITE_WEIGHT_GRAD);
      f = [=](device_stream_t const &s) {
        check_ffk(ffk_mha_forward(s.require_gpu(), type, &d, qp, kp, vp, w, y, reserve, reserve_bytes), "MultiHeadAttention forward");
      };
      b = [=](device_stream_t const &s) {
        check_ffk(ffk_mha_backward(s.require_gpu(), type, &d, qp, dq, kp, dk, vp, dv, w, dw, dy, reserve, reserve_bytes, accumulate),
                  "MultiHeadAttention backward");
      };
    } else if (auto const *a = std::get_if<DropoutAttrs>(&oa)) {
      tensor_guid_t x = layer.inputs[0];
      int const type = dt(shape_of(x).data_type);
      int64_t const n = numel(x);
      float const rate = a->rate;
      uint64_t const seed = a->seed + (uint64_t)l;
      void *xp = val(x), *dx = grd_or_discard(x);
      int const accumulate = p.bwd.accumulate ? 1 : 0;
      f = [=](device_stream_t const &s) {
        check_ffk(ffk_dropout_forward(s.require_gpu(), type, xp, y, n, rate, seed, S->iteration * (uint64_t)n), "Dropout forward");
      };
      b = [=](device_stream_t const &s) {
        check_ffk(ffk_dropout_backward(s.require_gpu(), type, dy, dx, n, rate, seed, S->iteration * (uint64_t)n, accumulate),
                  "Dropout backward");
      };
      if (fused[l] == Fused::GELU_DROPOUT_TAIL) {
        // y = dropout(GELU(u)) from the GELU's input; the backward of both runs at the GELU
        void *u = val(cg.layers[partner[l]].inputs[0]);
        f = [=](device_stream_t const &s) {
          check_ffk(ffk_gelu_dropout_forward(s.require_gpu(), type, u, y, n, rate, seed, S->iteration * (uint64_t)n),
                    "GELU + Dropout forward");
        };
        b = [](device_stream_t const &) {};
      } else if (fused[l] == Fused::DROPOUT_ADD_HEAD) {
        f = [](device_stream_t const &) {};  // the add computes residual + dropout(x)
      }
      if (drop_bwd_by_ln[l]) b = [](device_stream_t const &) {};  // the LayerNorm behind the add has written dx
      if (drop_bias[l] >= 0) {
        size_t const lin = (size_t)drop_bias[l];
        LinearAttrs const &la = std::get<LinearAttrs>(cg.layers[lin].attrs.op_attrs);
        int64_t const out_dim = la.out_channels, batch = n / out_dim;
        std::shared_ptr<bool> const done = bias_done[lin];
        void *dbias = grd(cg.layers[lin].weights.at(1));
        int const acc_bias = plan[lin].bwd.accumulate_input.at(2) ? 1 : 0;
        void *lin_scratch = base + plan[lin].scratch.offset;
        size_t const lin_scratch_bytes = plan[lin].scratch_bytes;
        b = [=](device_stream_t const &s) {
          uint64_t const offset = S->iteration * (uint64_t)n;
          int const rc = ffk_dropout_backward_bias_grad(s.require_gpu(), type, dy, dx, batch, out_dim, dbias, acc_bias, lin_scratch,
                                                        lin_scratch_bytes, rate, seed, offset);
          *done = rc == FFK_OK;
          if (rc != FFK_ERR_UNSUPPORTED) return check_ffk(rc, "Dropout backward with bias gradient");
          check_ffk(ffk_dropout_backward(s.require_gpu(), type, dy, dx, n, rate, seed, offset, accumulate), "Dropout backward");
        };
      }
    } else if (auto const *a = std::get_if<ElementUnaryAttrs>(&oa)) {
      tensor_guid_t x = layer.inputs[0];
      int const type = dt(shape_of(x).data_type), op = static_cast<int>(a->op_type);
      int64_t const n = numel(x);
      float const scalar = a->scalar.value_or(0.0f);
      void *xp = val(x), *dx = grd_or_discard(x);
      int const accumulate = p.bwd.accumulate ? 1 : 0;
      f = [=](device_stream_t const &s) {
        check_ffk(ffk_element_unary_forward(s.require_gpu(), type, op, scalar, xp, y, n), "ElementUnary forward");
      };
      b = [=](device_stream_t const &s) {
        check_ffk(ffk_element_unary_backward(s.require_gpu(), type, op, scalar, y, dy, xp, dx, n, accumulate), "ElementUnary backward");
      };
      if (fused[l] == Fused::GELU_DROPOUT_HEAD) {
        size_t const d = partner[l];
        DropoutAttrs const &da = std::get<DropoutAttrs>(cg.layers[d].attrs.op_attrs);
        float const rate = da.rate;
        uint64_t const seed = da.seed + (uint64_t)d;
        void *d_out = grd(cg.layers[d].outputs.at(0));
        f = [](device_stream_t const &) {};  // the Dropout computes dropout(GELU(x))
        if (gelu_linear[l] >= 0) {
          b = [](device_stream_t const &) {};  // the Linear that reads the Dropout's output has written dx
        } else if (p.bwd.has_backward) {
          b = [=](device_stream_t const &s) {
            check_ffk(ffk_dropout_gelu_backward(s.require_gpu(), type, d_out, xp, dx, n, rate, seed, S->iteration * (uint64_t)n),
                      "Dropout + GELU backward");
          };
        }
      }
    } else if (auto const *a = std::get_if<ElementBinaryAttrs>(&oa)) {
      tensor_guid_t lhs = layer.inputs[0], rhs = layer.inputs[1];
      int const type = dt(shape_of(out).data_type), op = static_cast<int>(a->type);
      int64_t const n = numel(out), nl = numel(lhs), nr = numel(rhs);
      void *lp = val(lhs), *rp = val(rhs), *dl = grd_or_discard(lhs), *dr = grd_or_discard(rhs);
      int const accumulate = p.bwd.accumulate ? 1 : 0;
      f = [=](device_stream_t const &s) {
        check_ffk(ffk_element_binary_forward(s.require_gpu(), type, op, lp, rp, y, n, nl, nr), "ElementBinary forward");
      };
      if (fused[l] == Fused::DROPOUT_ADD_TAIL) {
        size_t const d = partner[l];
        ComputationGraph::Layer const &drop = cg.layers[d];
        DropoutAttrs const &da = std::get<DropoutAttrs>(drop.attrs.op_attrs);
        float const rate = da.rate;
        uint64_t const seed = da.seed + (uint64_t)d;
        void *dropped_in = val(drop.inputs[0]);
        void *residual = lhs == drop.outputs.at(0) ? rp : lp;
        f = [=](device_stream_t const &s) {
          check_ffk(ffk_dropout_add_forward(s.require_gpu(), type, dropped_in, residual, y, n, rate, seed, S->iteration * (uint64_t)n),
                    "Dropout + add forward");
        };
        if (sum_linear[l] >= 0) f = [](device_stream_t const &) {};  // the Linear has written residual + dropout(Linear)
        if (add_fwd_by_ln[l]) f = [](device_stream_t const &) {};    // the LayerNorm that reads the sum computes it
      }
      if (p.bwd.add_by_alias) {
        // operands whose gradient is dy's own memory need nothing; the others get grad += dy
        // ... or, where this add is the first of them to run, grad = dy
        // ... and nothing where a LayerNorm that reads the operand takes dy as its residual
        void *add_l = has_grad[lhs.raw] && alias_of[lhs.raw] < 0 && deferred_to_ln[lhs.raw] < 0 ? grd(lhs) : nullptr;
        void *add_r = has_grad[rhs.raw] && alias_of[rhs.raw] < 0 && deferred_to_ln[rhs.raw] < 0 ? grd(rhs) : nullptr;
        bool const store_l = add_l != nullptr && !adds_here(lhs, l), store_r = add_r != nullptr && !adds_here(rhs, l);
        b = [=](device_stream_t const &s) {
          for (int side = 0; side < 2; side++) {
            void *g = side == 0 ? add_l : add_r;
            if (g == nullptr) continue;
            if (side == 0 ? store_l : store_r) {
              check_ffk(ffk_cast_forward(s.require_gpu(), type, type, dy, g, n), "ElementBinary backward");
            } else {
              check_ffk(ffk_element_binary_forward(s.require_gpu(), type, FFK_OP_EW_ADD, g, dy, g, n, n, n), "ElementBinary backward");
            }
          }
        };
      } else {
        b = [=](device_stream_t const &s) {
          check_ffk(ffk_element_binary_backward(s.require_gpu(), type, op, dy, lp, rp, dl, dr, n, accumulate), "ElementBinary backward");
        };
      }
    } else if (auto const *a = std::get_if<SoftmaxAttrs>(&oa)) {
      tensor_guid_t x = layer.inputs[0];
      int const type = dt(shape_of(x).data_type);
      int nd = get_num_dims(shape_of(x).dims), dim = a->dim < 0 ? nd + a->dim : a->dim;
      int64_t outer = 1, inner = 1;
      for (int i = 0; i < dim; i++) outer *= shape_of(x).dims.ff_ordered[i];
      for (int i = dim + 1; i < nd; i++) inner *= shape_of(x).dims.ff_ordered[i];
      int64_t const size = shape_of(x).dims.ff_ordered[dim], n = numel(x);
      void *xp = val(x), *dx = grd_or_discard(x);
      bool const via_scratch = p.bwd.softmax_via_scratch;
      f = [=](device_stream_t const &s) {
        check_ffk(ffk_softmax_forward(s.require_gpu(), type, xp, y, outer, size, inner), "Softmax forward");
      };
      // The cross-entropy loss kernels write (p - label) * scale into the gradient of the
      // probabilities they are given (loss_function_kernels.cu:21-57): for a softmax output
      // that is already the gradient of the softmax INPUT, which is why the reference's
      // Softmax backward is a copy (softmax_kernels.cu:68-78).  Such a softmax passes the
      // gradient through; every other softmax gets the true gradient.
      bool feeds_cross_entropy = false;
      if (loss.has_value() && loss->logit_tensor == layer.outputs[0]) {
        LossFunction const kind = get_loss_function(loss->loss_attrs);
        feeds_cross_entropy = kind == LossFunction::SPARSE_CATEGORICAL_CROSSENTROPY || kind == LossFunction::CATEGORICAL_CROSSENTROPY;
      }
      if (feeds_cross_entropy) {
        b = [=](device_stream_t const &s) {
          if (via_scratch) {
            check_ffk(ffk_element_binary_forward(s.require_gpu(), type, FFK_OP_EW_ADD, dx, dy, dx, n, n, n), "Softmax backward");
          } else {
            check_ffk(ffk_softmax_backward_copy(s.require_gpu(), type, dy, dx, (size_t)n), "Softmax backward");
          }
        };
      } else {
        b = [=](device_stream_t const &s) {
          check_ffk(ffk_softmax_backward(s.require_gpu(), type, y, dy, via_scratch ? scratch : dx, outer, size, inner), "Softmax backward");
          if (via_scratch) {
            check_ffk(ffk_element_binary_forward(s.require_gpu(), type, FFK_OP_EW_ADD, dx, scratch, dx, n, n, n), "Softmax backward");
          }
        };
      }
    } else if (auto const *a = std::get_if<EmbeddingAttrs>(&oa)) {
      tensor_guid_t x = layer.inputs[0];
      int const itype = dt(shape_of(x).data_type), otype = dt(a->data_type), aggr = aggr_code(a->aggr);
      int64_t const bag = a->aggr.has_value() ? dim_at_idx(shape_of(x).dims, -1) : 1;
      int64_t const bags = numel(x) / bag, dim = a->out_channels, entries = a->num_entries;
      void *xp = val(x), *w = val(layer.weights[0]);
      float *dw = static_cast<float *>(grd(layer.weights[0]));
      f = [=](device_stream_t const &s) {
        check_ffk(ffk_embedding_forward(s.require_gpu(), itype, FFK_FLOAT, otype, xp, y, w, aggr, bags, bag, dim, entries), "Embedding forward");
      };
      b = [=](device_stream_t const &s) {
        check_ffk(ffk_embedding_backward(s.require_gpu(), itype, otype, xp, dy, dw, aggr, bags, bag, dim, entries, 0,
                                         ws_bytes ? scratch : nullptr, ws_bytes),
                  "Embedding backward");
      };
    } else if (auto const *a = std::get_if<ConcatAttrs>(&oa)) {
      int const type = dt(shape_of(out).data_type);
      int nd = get_num_dims(shape_of(out).dims), axis = a->axis < 0 ? nd + a->axis : a->axis;
      int64_t blocks = 1;
      for (int i = 0; i < axis; i++) blocks *= shape_of(out).dims.ff_ordered[i];
      std::vector<void const *> in_ptrs;
      std::vector<void *> grad_ptrs;
      std::vector<int64_t> blks;
      for (tensor_guid_t t : layer.inputs) {
        in_ptrs.push_back(val(t));
        grad_ptrs.push_back(grd_or_discard(t));
        blks.push_back(numel(t) / blocks);
      }
      int const parts = (int)layer.inputs.size(), accumulate = p.bwd.accumulate ? 1 : 0;
      f = [=](device_stream_t const &s) {
        check_ffk(ffk_concat_forward(s.require_gpu(), type, y, in_ptrs.data(), blks.data(), parts, blocks), "Concat forward");
      };
      b = [=](device_stream_t const &s) {
        check_ffk(ffk_concat_backward(s.require_gpu(), type, dy, grad_ptrs.data(), blks.data(), parts, blocks, accumulate),
                  "Concat backward");
      };
    } else if (auto const *a = std::get_if<TransposeAttrs>(&oa)) {
      tensor_guid_t x = layer.inputs[0];
      int const type = dt(shape_of(x).data_type), nd = get_num_dims(shape_of(x).dims);
      std::vector<int64_t> const dims = shape_of(x).dims.ff_ordered;
      std::vector<int> const perm = a->permutation;
      void *xp = val(x), *dx = grd_or_discard(x);
      int const accumulate = p.bwd.accumulate ? 1 : 0;
      f = [=](device_stream_t const &s) {
        check_ffk(ffk_transpose_forward(s.require_gpu(), type, xp, y, nd, dims.data(), perm.data()), "Transpose forward");
      };
      b = [=](device_stream_t const &s) {
        check_ffk(ffk_transpose_backward(s.require_gpu(), type, dy, dx, nd, dims.data(), perm.data(), accumulate),
                  "Transpose backward");
      };
    } else if (std::get_if<ReshapeAttrs>(&oa)) {
      // the same elements in the same order: a flat copy forward, a flat copy or add backward
      tensor_guid_t x = layer.inputs[0];
      int const type = dt(shape_of(x).data_type);
      int64_t const n = numel(x);
      int64_t const flat = n;
      int const one = 0;
      void *xp = val(x), *dx = grd_or_discard(x);
      int const accumulate = p.bwd.accumulate ? 1 : 0;
      f = [=](device_stream_t const &s) {
        check_ffk(ffk_transpose_forward(s.require_gpu(), type, xp, y, 1, &flat, &one), "Reshape forward");
      };
      b = [=](device_stream_t const &s) {
        check_ffk(ffk_transpose_backward(s.require_gpu(), type, dy, dx, 1, &flat, &one, accumulate), "Reshape backward");
      };
    } else if (auto const *a = std::get_if<GatherAttrs>(&oa)) {
      tensor_guid_t x = layer.inputs[0], index = layer.inputs[1];
      int const type = dt(shape_of(x).data_type), itype = dt(shape_of(index).data_type);
      int nd = get_num_dims(shape_of(x).dims), d = a->dim < 0 ? nd + a->dim : a->dim;
      int64_t outer = 1, stride = 1;
      for (int i = 0; i < d; i++) outer *= shape_of(x).dims.ff_ordered[i];
      for (int i = d + 1; i < nd; i++) stride *= shape_of(x).dims.ff_ordered[i];
      int64_t const in_dim = shape_of(x).dims.ff_ordered[d], out_dim = shape_of(index).dims.ff_ordered[d];
      void *xp = val(x), *ip = val(index);
      float *dx = static_cast<float *>(grd(x));
      f = [=](device_stream_t const &s) {
        check_ffk(ffk_gather_forward(s.require_gpu(), type, itype, xp, ip, y, outer, in_dim, out_dim, stride), "Gather forward");
      };
      b = [=](device_stream_t const &s) {
        if (dx != nullptr) {
          check_ffk(ffk_gather_backward(s.require_gpu(), itype, static_cast<float const *>(dy), ip, dx, outer, in_dim,
                                        out_dim, stride),
                    "Gather backward");
        }
      };
    } else if (std::get_if<CastAttrs>(&oa)) {
      tensor_guid_t x = layer.inputs[0];
      int const itype = dt(shape_of(x).data_type), otype = dt(shape_of(out).data_type);
      int64_t const n = numel(x);
      void *xp = val(x), *dx = grd(x);
      f = [=](device_stream_t const &s) { check_ffk(ffk_cast_forward(s.require_gpu(), itype, otype, xp, y, n), "Cast forward"); };
      b = [=](device_stream_t const &s) { check_ffk(ffk_cast_backward(s.require_gpu(), otype, itype, dy, dx, n), "Cast backward"); };
    } else {
      bad("operator has no task implementation");
    }
    fwd.push_back(DynamicNodeInvocation{DynamicTaskType::FWD, id, f});
    if (p.bwd.has_backward) bwd.push_back(DynamicNodeInvocation{DynamicTaskType::BWD, id, b});
  }

  // -- LOSS (loss_functions.cc:24-150)
  std::vector<DynamicNodeInvocation> order = fwd;
  if (loss.has_value()) {
    TensorShape const &ls = shape_of(loss->logit_tensor);
    GenericTensorAccessorW const label = loss->label_tensor;
    if (label.device_type != DeviceType::GPU) bad("the label tensor is not device-resident");
    if (get_num_dims(ls.dims) < 2) bad("the logit tensor is [batch, classes]");
    int const batch_size = (int)dim_at_idx(ls.dims, -2);
    int const num_classes = (int)dim_at_idx(ls.dims, -1);
    int64_t const volume = get_num_elements(ls.dims);
    float *logit = static_cast<float *>(val(loss->logit_tensor));
    float *dlogit = static_cast<float *>(grd(loss->logit_tensor));
    LossFunction const kind = get_loss_function(loss->loss_attrs);
    std::function<void(device_stream_t const &)> f;
    if (kind == LossFunction::SPARSE_CATEGORICAL_CROSSENTROPY) {
      if (label.shape.data_type != DataType::INT32) bad("sparse labels are INT32");
      int k = 1;
      if (std::get<SparseCategoricalCrossEntropyLossAttrs>(loss->loss_attrs).replace_labels) {
        k = (int)(dim_at_idx(ls.dims, 0) / dim_at_idx(label.shape.dims, 0));
      }
      if ((int64_t)k * get_num_elements(label.shape.dims) != volume / num_classes) bad("label count does not match the logits");
      int const samples = (int)(volume / num_classes);
      float const scale = 1.0f / batch_size;
      int const *lab = static_cast<int const *>(label.ptr);
      f = [=](device_stream_t const &s) {
        check_ffk(ffk_sparse_categorical_crossentropy_loss_backward(s.require_gpu(), dlogit, logit, lab, volume, volume, samples,
                                                                    num_classes, k, scale),
                  "SparseCategoricalCrossEntropyLoss backward");
      };
    } else {
      if (kind != LossFunction::IDENTITY && (label.shape.data_type != DataType::FLOAT || get_num_elements(label.shape.dims) != volume)) {
        bad("the label tensor must match the FLOAT logits");
      }
      float const *lab = static_cast<float const *>(label.ptr);
      if (kind == LossFunction::CATEGORICAL_CROSSENTROPY) {
        float const scale = 1.0f / batch_size;
        f = [=](device_stream_t const &s) {
          check_ffk(ffk_categorical_crossentropy_loss_backward(s.require_gpu(), dlogit, logit, lab, volume, volume, scale),
                    "CategoricalCrossEntropyLoss backward");
        };
      } else if (kind == LossFunction::MEAN_SQUARED_ERROR_AVG_REDUCE) {
        float const scale = 2.0f / (float)volume;
        f = [=](device_stream_t const &s) {
          check_ffk(ffk_mean_squared_error_avg_loss_backward(s.require_gpu(), dlogit, logit, lab, volume, volume, scale),
                    "MeanSquaredErrorAvgLoss backward");
        };
      } else if (kind == LossFunction::IDENTITY) {
        float const scale = 1.0f / batch_size;
        f = [=](device_stream_t const &s) {
          check_ffk(ffk_identity_loss_backward(s.require_gpu(), dlogit, logit, volume, volume, scale), "IdentityLoss backward");
        };
      } else {
        bad("unsupported loss function");  // the reference panics on MEAN_SQUARED_ERROR_SUM_REDUCE too
      }
    }
    order.push_back(DynamicNodeInvocation{DynamicTaskType::LOSS, layer_guid_t{-1}, f});
  }
  for (auto it = bwd.rbegin(); it != bwd.rend(); ++it) order.push_back(*it);

  // -- UPD, one invocation per weight (optimizer.cc:10-108).  The first member of a
  // weight group updates the whole group with one launch; the invocations of the
  // other members are empty.
  auto make_update = [S](int grad_type, void *g, int64_t n, float *w32, float *v, float *m, void *wlow) {
    return [=](device_stream_t const &stream) {
      if (auto const *sgd = std::get_if<SGDOptimizerAttrs>(&S->optimizer_attrs)) {
        check_ffk(ffk_sgd_update(stream.require_gpu(), grad_type, (float)sgd->lr, (float)sgd->momentum, sgd->nesterov,
                                 (float)sgd->weight_decay, g, n, 1, w32, v, wlow),
                  "SGD update");
      } else {
        AdamOptimizerAttrs const &adam_attrs = std::get<AdamOptimizerAttrs>(S->optimizer_attrs);
        check_ffk(ffk_adam_update(stream.require_gpu(), grad_type, (float)adam_attrs.alpha_t, (float)adam_attrs.beta1,
                                  (float)adam_attrs.beta2, (float)adam_attrs.weight_decay, (float)adam_attrs.epsilon, g, n, 1,
                                  w32, v, m, wlow),
                  "Adam update");
      }
    };
  };
  for (size_t t = 0; t < T; t++) {
    if (!is_weight[t] || !has_grad[t]) continue;
    std::function<void(device_stream_t const &)> f = [](device_stream_t const &) {};
    if (group_of[t] >= 0) {
      WeightGroup const &g = groups[(size_t)group_of[t]];
      if (g.members.front() == t) {
        bool const lowp = g.type == DataType::BF16;
        f = make_update(dt(g.type), base + g.grad.offset, (int64_t)g.elems,
                        reinterpret_cast<float *>(base + (lowp ? g.master.offset : g.value.offset)),
                        g.v.bytes ? reinterpret_cast<float *>(base + g.v.offset) : nullptr,
                        g.m.bytes ? reinterpret_cast<float *>(base + g.m.offset) : nullptr,
                        lowp ? static_cast<void *>(base + g.value.offset) : nullptr);
      }
    } else {
      TensorShape const &s = cg.tensors[t].shape;
      bool const lowp = s.data_type == DataType::BF16;
      f = make_update(dt(s.data_type), st->grad[t]->ptr, get_num_elements(s.dims),
                      static_cast<float *>(lowp ? st->master[t]->ptr : st->value[t].ptr),
                      st->opt_v[t].has_value() ? static_cast<float *>(st->opt_v[t]->ptr) : nullptr,
                      st->opt_m[t].has_value() ? static_cast<float *>(st->opt_m[t]->ptr) : nullptr,
                      lowp ? st->value[t].ptr : nullptr);
    }
    order.push_back(DynamicNodeInvocation{DynamicTaskType::UPD, cg.tensors[t].source, f});
  }
  st->order = order;
  return ComputationGraphInstance{st};
}

// ---- execution ------------------------------------------------------------------

static LayerTimings execute(ComputationGraphInstance const &instance, ProfilingSettings const &profiling,
                            std::function<bool(DynamicTaskType)> const &selected) {
  LayerTimings result;
  bool cleared = false, masters = false, collecting = false;
  // The last step of every bias and LayerNorm parameter gradient is collected over the backward
  // pass and run as one launch behind it (not when invocations are repeated for timing).
  bool const collect = profiling.warmup_iters == 0 && profiling.measure_iters == 0;
  auto end_collection = [&] {
    if (collecting) check_ffk(ffk_column_reductions_end(get_gpu_device_stream().require_gpu()), "column reductions");
    collecting = false;
  };
  try {
    for (DynamicNodeInvocation const &inv : instance.get_execution_order()) {
      if (!selected(inv.task_type)) continue;
      if (!cleared && (inv.task_type == DynamicTaskType::LOSS || inv.task_type == DynamicTaskType::BWD)) {
        instance.clear_accumulated_gradients(get_gpu_device_stream());
        cleared = true;
      }
      if (inv.task_type == DynamicTaskType::BWD && collect && !collecting) {
        check_ffk(ffk_column_reductions_begin(), "column reductions");
        collecting = true;
      }
      if (inv.task_type == DynamicTaskType::UPD) end_collection();
      if (!masters && inv.task_type == DynamicTaskType::UPD) {
        if (!instance.state->masters_valid) instance.sync_master_weights();
        masters = true;
      }
      result[inv.layer_guid] = profiling_wrapper(inv.run, profiling, DeviceType::GPU);
    }
    end_collection();
  } catch (...) {
    if (collecting) ffk_column_reductions_end(get_gpu_device_stream().require_gpu());
    throw;
  }
  return result;
}

LayerTimings perform_all_passes_for_computation_graph_instance(ComputationGraphInstance &instance,
                                                               ProfilingSettings const &profiling, device_handle_t const &,
                                                               device_id_t) {
  LayerTimings r = execute(instance, profiling, [](DynamicTaskType) { return true; });
  instance.update_optimizer_attrs_for_next_iter();
  return r;
}
LayerTimings perform_forward_pass_for_computation_graph_instance(ComputationGraphInstance const &instance,
                                                                 ProfilingSettings const &profiling, device_handle_t const &,
                                                                 device_id_t) {
  return execute(instance, profiling, [](DynamicTaskType t) { return t == DynamicTaskType::FWD; });
}
LayerTimings perform_backward_pass_for_computation_graph_instance(ComputationGraphInstance const &instance,
                                                                  ProfilingSettings const &profiling, device_handle_t const &,
                                                                  device_id_t) {
  return execute(instance, profiling, [](DynamicTaskType t) { return t == DynamicTaskType::BWD; });
}
void perform_update_pass_for_computation_graph_instance(ComputationGraphInstance &instance, ProfilingSettings const &profiling,
                                                        device_handle_t const &, device_id_t) {
  execute(instance, profiling, [](DynamicTaskType t) { return t == DynamicTaskType::UPD; });
  instance.update_optimizer_attrs_for_next_iter();
}

}  // namespace FlexFlow
