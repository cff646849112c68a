// Times the step driver on one training step of the encoder layer the headline
// figure is quoted on (pre-LN, GELU, dropout 0.1, batch 8 x 512 tokens, d_model
// 1024, 16 heads, FFN 4096, BF16): forward, backward and SGD update, operator by
// operator, the way the reference's local-execution backend drives lib/kernels
// (lib/local-execution/src/local-execution/computation_graph_instance.cc:
// perform_all_passes_for_computation_graph_instance).
//   step_bench [steps]
#include "ffk.h"
#include "kernels/allocation.h"
#include "kernels/profiling.h"
#include "local-execution/computation_graph_instance.h"
#include "pcg/computation_graph_builder.h"
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <vector>

using namespace FlexFlow;

static TensorShape shape(std::vector<int64_t> dims, DataType dtype) { return TensorShape{TensorDims{dims}, dtype}; }

// round-to-nearest-even BF16 bits of a finite float
static uint16_t bf16_bits(float v) {
  uint32_t u;
  memcpy(&u, &v, 4);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

// fills a BF16 device accessor with U(lo, hi) values
static void fill_uniform(Allocator &gpu, GenericTensorAccessorW const &dst, unsigned seed, float lo, float hi) {
  if (dst.shape.data_type != DataType::BF16) throw std::runtime_error("step_bench: the layer is BF16 throughout");
  Allocator cpu = create_local_cpu_memory_allocator();
  GenericTensorAccessorW h = cpu.allocate_tensor(dst.shape);
  size_t const n = (size_t)get_num_elements(dst.shape.dims);
  std::mt19937 gen(seed);
  std::uniform_real_distribution<float> dist(lo, hi);
  uint16_t *p = static_cast<uint16_t *>(h.ptr);
  for (size_t i = 0; i < n; i++) p[i] = bf16_bits(dist(gen));
  (void)gpu;
  copy_accessor_data_to_l_from_r(dst, h);
}

static void run(int steps) {
  ManagedPerDeviceFFHandle managed = initialize_single_gpu_handle(1 << 20, true);
  device_handle_t handle = device_handle_t_from_managed_ff_handle(managed);
  Allocator gpu = create_local_cuda_memory_allocator();
  int const B = 8, S = 512, E = 1024, H = 16, FF = 4096;
  ComputationGraphBuilder cgb;
  tensor_guid_t x = cgb.create_input(shape({B, S, E}, DataType::BF16), CreateGrad::YES);
  tensor_guid_t n1 = cgb.layer_norm(x, {-1}, true, 1e-5f);
  tensor_guid_t att = cgb.multihead_attention(n1, n1, n1, E, H, E / H, E / H, 0.0f, false, false, false, std::nullopt, 0.125f);
  tensor_guid_t r1 = cgb.add(x, cgb.dropout(att, 0.1f));
  tensor_guid_t n2 = cgb.layer_norm(r1, {-1}, true, 1e-5f);
  tensor_guid_t f1 = cgb.dense(n2, FF, Activation::GELU, true);
  tensor_guid_t f2 = cgb.dense(cgb.dropout(f1, 0.1f), E, std::nullopt, true);
  tensor_guid_t out = cgb.add(r1, cgb.dropout(f2, 0.1f));
  device_id_t dev = make_device_id_t_from_idx(0, DeviceType::GPU);
  ComputationGraphInstance inst = create_computation_graph_instance(
      cgb.computation_graph, OptimizerAttrs{SGDOptimizerAttrs{1e-5, 0.0, false, 0.0}}, std::nullopt, {}, gpu,
      ProfilingSettings{0, 0}, handle, dev);
  unsigned seed = 1;
  for (size_t t = 0; t < cgb.computation_graph.tensors.size(); t++) {
    auto const &src = cgb.computation_graph.layers[cgb.computation_graph.tensors[t].source.raw];
    bool const weight = std::holds_alternative<WeightAttrs>(src.attrs.op_attrs);
    if (!weight && tensor_guid_t{(int)t} != x) continue;
    fill_uniform(gpu, inst.get_tensor_accessor(tensor_guid_t{(int)t}), seed++, -0.05f, 0.05f);
  }
  // a small output gradient: with a gradient of order one per element and no loss to normalise
  // it, a few SGD steps drive the weights to infinity
  fill_uniform(gpu, *inst.get_gradient_accessor(out), 99, -1e-3f, 1e-3f);
  device_stream_t stream = get_gpu_device_stream();
  auto step = [&] { perform_all_passes_for_computation_graph_instance(inst, ProfilingSettings{0, 0}, handle, dev); };
  // untimed first: the shader clock takes tens of milliseconds of sustained load to reach the
  // state it then holds, and steps timed inside that ramp run 5% slow
  for (int i = 0; i < 400; i++) step();
  ffEvent_t t0, t1;
  check_ffk(ffk_event_create(&t0), "event");
  check_ffk(ffk_event_create(&t1), "event");
  check_ffk(ffk_event_record(t0, stream.require_gpu()), "event");
  for (int i = 0; i < steps; i++) step();
  check_ffk(ffk_event_record(t1, stream.require_gpu()), "event");
  check_ffk(ffk_event_synchronize(t1), "event");
  float ms = 0;
  check_ffk(ffk_event_elapsed_ms(t0, t1, &ms), "event");
  {
    // the numbers are only meaningful on healthy data: a step that has diverged runs on NaNs,
    // which toggle no bits and let the chip clock higher
    Allocator cpu = create_local_cpu_memory_allocator();
    GenericTensorAccessorW h = copy_tensor_accessor_w(inst.get_tensor_accessor(out), cpu);
    size_t const n = (size_t)get_num_elements(h.shape.dims);
    uint16_t const *p = static_cast<uint16_t const *>(h.ptr);
    size_t bad = 0;
    double sum = 0;
    for (size_t i = 0; i < n; i++) {
      uint32_t u = (uint32_t)p[i] << 16;
      float v;
      memcpy(&v, &u, 4);
      bad += !std::isfinite(v);
      sum += std::isfinite(v) ? std::fabs(v) : 0.0;
    }
    printf("output after the run: %zu non-finite of %zu, mean |y| %.4f\n", bad, n, sum / (double)n);
  }
  int const invocations = (int)inst.get_execution_order().size();
  printf("step driver, encoder layer B8 S512 d1024 h16 ffn4096 bf16, FWD+BWD+SGD: %.3f ms/step over %d steps, "
         "%d invocations, %.1f MiB placed, %.2f M tokens/s\n",
         ms / steps, steps, invocations, inst.bytes_allocated() / 1048576.0, B * S / (ms / steps) / 1e3);
}

int main(int argc, char **argv) {
  int const steps = argc > 1 ? atoi(argv[1]) : 20;
  if (steps <= 0) {
    printf("usage: step_bench [steps]\n");
    return 2;
  }
  try {
    run(steps);
  } catch (std::exception const &e) {
    printf("step_bench failed: %s\n", e.what());
    return 1;
  }
  return 0;
}
