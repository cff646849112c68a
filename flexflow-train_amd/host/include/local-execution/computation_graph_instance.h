// One training step over a ComputationGraph on one device (reference:
// lib/local-execution/include/local-execution/computation_graph_instance.h:22-89,
// loss_config.dtg.toml; lib/pcg/include/pcg/optimizer_attrs.dtg.toml,
// optimizers/{sgd,adam}_optimizer_attrs.dtg.toml; lib/op-attrs/include/op-attrs/
// ops/loss_functions/).
//
// create_computation_graph_instance expands every layer into a FWD and a BWD
// invocation, appends the LOSS invocation and one UPD invocation per weight,
// places all tensors, and initialises per-operator state.  The
// perform_*_pass functions then replay that list; nothing is allocated while
// stepping.  Differences from the reference that a caller can see:
//  * gradients are cleared by the instance: it knows, per gradient tensor,
//    whether its only producer can overwrite it (then it is never cleared) or
//    whether several producers add into it; then the producer that runs first
//    in the backward pass stores where it can, and otherwise the gradient sits
//    in a region that one fill clears before the backward pass.  The reference leaves gradient
//    memory as allocated and lets every GPU backward add into it.
//  * weights of BF16 data type are trained with an fp32 master copy that the
//    update kernel rounds into the BF16 tensor (the master is taken from the
//    BF16 values at the first update, or when sync_master_weights is called).
//  * a dropout layer's mask differs per layer and per iteration: seed + layer
//    index, offset = iteration * elements.
//  * two neighbouring operators run as one kernel where the library has one
//    that produces the same bits: GELU -> Dropout (forward and backward) and
//    Dropout -> element-wise add (forward).  The tensor between them must have
//    no other consumer; it is then never written (get_tensor_accessor on it
//    returns memory nobody filled).  A BF16 Linear without activation whose
//    output only feeds such a Dropout -> add pair writes the sum from its
//    GEMM (its own output is never written); one whose input only comes from
//    such a GELU -> Dropout pair writes the gradient of the GELU's input from
//    its input-gradient GEMM (the gradient of its own input is never written).
//    ffk_set_option(FFK_OPTION_LAYER_UNFUSED, 1) before creation keeps one
//    kernel per operator.
//  * the backward of an element-wise add copies nothing: an operand whose
//    gradient has no other producer shares the output gradient's memory
//    (get_gradient_accessor of both returns the same pointer), an operand that
//    other operators also add into gets grad += dy.
//  * the weights the instance places itself are grouped by data type: value,
//    gradient, master and moments of a group lie in parallel arrays, and the
//    UPD invocation of the group's first weight updates all of them with one
//    launch (the UPD invocations of the other members are empty).  A weight
//    bound to caller memory is updated by its own launch.
#pragma once
#include "kernels/accessor.h"
#include "kernels/allocation.h"
#include "kernels/device_stream_t.h"
#include "kernels/profiling.h"
#include "pcg/computation_graph.h"
#include <memory>
#include <unordered_map>

namespace FlexFlow {

enum class LossFunction {
  CATEGORICAL_CROSSENTROPY,
  SPARSE_CATEGORICAL_CROSSENTROPY,
  MEAN_SQUARED_ERROR_AVG_REDUCE,
  MEAN_SQUARED_ERROR_SUM_REDUCE,
  IDENTITY
};
struct SparseCategoricalCrossEntropyLossAttrs { bool replace_labels; };
struct NonconfigurableLossAttrs { LossFunction loss_type; };
using LossAttrs = std::variant<SparseCategoricalCrossEntropyLossAttrs, NonconfigurableLossAttrs>;
LossFunction get_loss_function(LossAttrs const &);

struct LossConfig {
  LossAttrs loss_attrs;
  GenericTensorAccessorW label_tensor;
  tensor_guid_t logit_tensor;
};

struct SGDOptimizerAttrs {
  double lr, momentum;
  bool nesterov;
  double weight_decay;
};
struct AdamOptimizerAttrs {
  double alpha, beta1, beta2, weight_decay, alpha_t, beta_t, beta2_t, epsilon;
};
using OptimizerAttrs = std::variant<SGDOptimizerAttrs, AdamOptimizerAttrs>;
// lib/pcg/src/pcg/optimizer_attrs.cc:6-26
OptimizerAttrs get_optimizer_attrs_for_next_iter(OptimizerAttrs const &);

struct device_id_t {
  int idx;
  DeviceType device_type;
};
inline device_id_t make_device_id_t_from_idx(int idx, DeviceType t) { return device_id_t{idx, t}; }

enum class DynamicTaskType { FWD, BWD, UPD, LOSS };

struct DynamicNodeInvocation {
  DynamicTaskType task_type;
  layer_guid_t layer_guid;
  std::function<void(device_stream_t const &)> run;
};

struct ComputationGraphInstance {
  struct State;
  ComputationGraphInstance() = delete;
  explicit ComputationGraphInstance(std::shared_ptr<State> state);

  std::vector<DynamicNodeInvocation> const &get_execution_order() const;
  Allocator &get_allocator() const;
  OptimizerAttrs const &get_optimizer_attrs() const;
  void update_optimizer_attrs_for_next_iter();
  std::optional<GenericTensorAccessorR> get_loss_tensor_accessor() const;

  // The placed tensors, for filling inputs and weights and reading results.
  GenericTensorAccessorW get_tensor_accessor(tensor_guid_t) const;
  std::optional<GenericTensorAccessorW> get_gradient_accessor(tensor_guid_t) const;
  // fp32 master / optimizer tensors of a weight (nullopt when there is none)
  std::optional<GenericTensorAccessorW> get_master_weight_accessor(tensor_guid_t) const;
  // Re-reads the fp32 masters from the BF16 weight tensors.
  void sync_master_weights() const;
  // Clears what the backward pass adds into (done by the pass functions themselves).
  void clear_accumulated_gradients(device_stream_t const &) const;
  size_t bytes_allocated() const;

  std::shared_ptr<State> state;
};

ComputationGraphInstance create_computation_graph_instance(
    ComputationGraph const &cg, OptimizerAttrs const &optimizer_attrs, std::optional<LossConfig> const &loss,
    std::unordered_map<tensor_guid_t, GenericTensorAccessorW> const &input_tensors, Allocator &allocator,
    ProfilingSettings const &profiling_settings, device_handle_t const &device_handle, device_id_t device_idx);

using LayerTimings = std::unordered_map<layer_guid_t, std::optional<milliseconds_t>>;

// FWD of every layer in order, LOSS, BWD in reverse order, UPD of every weight,
// then the optimizer attrs advance (computation_graph_instance.cc:140-157).
LayerTimings perform_all_passes_for_computation_graph_instance(ComputationGraphInstance &instance,
                                                               ProfilingSettings const &profiling_settings,
                                                               device_handle_t const &ff_handle,
                                                               device_id_t device_idx);
LayerTimings perform_forward_pass_for_computation_graph_instance(ComputationGraphInstance const &instance,
                                                                 ProfilingSettings const &profiling_settings,
                                                                 device_handle_t const &ff_handle,
                                                                 device_id_t device_idx);
// BWD invocations only: the logit gradient is taken as it stands.
LayerTimings perform_backward_pass_for_computation_graph_instance(ComputationGraphInstance const &instance,
                                                                  ProfilingSettings const &profiling_settings,
                                                                  device_handle_t const &ff_handle,
                                                                  device_id_t device_idx);
void perform_update_pass_for_computation_graph_instance(ComputationGraphInstance &instance,
                                                        ProfilingSettings const &profiling_settings,
                                                        device_handle_t const &ff_handle, device_id_t device_idx);

}  // namespace FlexFlow
