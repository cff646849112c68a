// Tests of the host mirror, written the way the reference's kernel tests are
// (lib/kernels/test/src: allocate through an Allocator, fill accessors, call
// the entry point, copy back, compare).  The CPU oracle is the checker.
//   test_host --cpu   host-only checks (no device needed)
//   test_host --gpu   every operator entry point on the device
#include "ffk_oracle.h"
#include "kernels/allocation.h"
#include "kernels/attention_kernels.h"
#include "kernels/cast_kernels.h"
#include "kernels/concat_kernels.h"
#include "kernels/dropout_kernels.h"
#include "kernels/element_kernels.h"
#include "kernels/embedding_kernels.h"
#include "kernels/layer_norm_kernels.h"
#include "kernels/linear_kernels.h"
#include "kernels/loss_function_kernels.h"
#include "kernels/optimizer_kernels.h"
#include "kernels/profiling.h"
#include "kernels/shape_kernels.h"
#include "kernels/softmax_kernels.h"
#include "ffk.h"
#include "local-execution/computation_graph_instance.h"
#include "pcg/computation_graph_builder.h"
#include <cmath>
#include <cstdio>
#include <cstring>
#include <functional>
#include <random>
#include <string>

using namespace FlexFlow;

// test_reference_includes.cc: a translation unit that uses only the reference's include lines
std::string reference_style_translation_unit();

static int g_failed = 0, g_checks = 0;
#define CHECK(cond)                                                            \
  do {                                                                         \
    g_checks++;                                                                \
    if (!(cond)) {                                                             \
      g_failed++;                                                              \
      printf("  CHECK failed: %s (%s:%d)\n", #cond, __FILE__, __LINE__);       \
    }                                                                          \
  } while (0)
#define CHECK_THROWS(expr)                                                     \
  do {                                                                         \
    g_checks++;                                                                \
    bool threw__ = false;                                                      \
    try { (void)(expr); } catch (std::exception const &) { threw__ = true; }   \
    if (!threw__) {                                                            \
      g_failed++;                                                              \
      printf("  CHECK_THROWS failed: %s (%s:%d)\n", #expr, __FILE__, __LINE__);\
    }                                                                          \
  } while (0)

static void run(char const *name, std::function<void()> const &f) {
  printf("TEST_CASE %s\n", name);
  fflush(stdout);
  int const failed_before = g_failed;
  try {
    f();
  } catch (std::exception const &e) {
    g_failed++;
    printf("  exception: %s\n", e.what());
  }
  // one line per case, so a harness can report every case on its own
  printf("CASE_RESULT %s\n", g_failed == failed_before ? "ok" : "FAILED");
  fflush(stdout);
}

static TensorShape shape(std::vector<int64_t> dims, DataType dtype) { return TensorShape{TensorDims{dims}, dtype}; }

static std::vector<float> random_vec(size_t n, unsigned seed, float lo = -1.0f, float hi = 1.0f) {
  std::mt19937 gen(seed);  // the reference's tests use std::mt19937(0) and U(-1, 1)
  std::uniform_real_distribution<float> dist(lo, hi);
  std::vector<float> v(n);
  for (auto &x : v) x = dist(gen);
  return v;
}

// device accessor filled from host floats (converted to the accessor's dtype)
static GenericTensorAccessorW device_accessor(Allocator &gpu, TensorShape const &s, std::vector<float> const &host) {
  Allocator cpu = create_local_cpu_memory_allocator();
  GenericTensorAccessorW h = cpu.allocate_tensor(s);
  size_t n = (size_t)get_num_elements(s.dims);
  if (s.data_type == DataType::FLOAT) {
    memcpy(h.ptr, host.data(), n * 4);
  } else if (s.data_type == DataType::BF16) {
    uint16_t *p = static_cast<uint16_t *>(h.ptr);
    for (size_t i = 0; i < n; i++) {
      float r = orc_round_bf16(host[i]);
      uint32_t u;
      memcpy(&u, &r, 4);
      p[i] = (uint16_t)(u >> 16);
    }
  } else {
    throw std::runtime_error("device_accessor: dtype");
  }
  GenericTensorAccessorW d = gpu.allocate_tensor(s);
  copy_accessor_data_to_l_from_r(d, h);
  return d;
}

static std::vector<float> to_host(GenericTensorAccessorW const &d) {
  Allocator cpu = create_local_cpu_memory_allocator();
  GenericTensorAccessorW h = copy_tensor_accessor_w(d, cpu);
  size_t n = (size_t)get_num_elements(d.shape.dims);
  std::vector<float> out(n);
  if (d.shape.data_type == DataType::FLOAT) {
    memcpy(out.data(), h.ptr, n * 4);
  } else {
    uint16_t const *p = static_cast<uint16_t const *>(h.ptr);
    for (size_t i = 0; i < n; i++) {
      uint32_t u = (uint32_t)p[i] << 16;
      memcpy(&out[i], &u, 4);
    }
  }
  return out;
}

static bool close(std::vector<float> const &a, std::vector<float> const &b, double rtol) {
  if (a.size() != b.size()) return false;
  double scale = 0;
  for (float v : b) scale = std::max(scale, (double)std::fabs(v));
  for (size_t i = 0; i < a.size(); i++) {
    if (std::fabs((double)a[i] - b[i]) > rtol * scale + rtol * std::fabs(b[i])) {
      printf("  mismatch at %zu: got %g want %g\n", i, a[i], b[i]);
      return false;
    }
  }
  return true;
}

static bool contains_non_zero(std::vector<float> const &v) {
  for (float x : v) if (x != 0.0f) return true;
  return false;
}

// ---------------------------------------------------------------------------
static void cpu_tests() {
  run("calculate_accessor_offset", [] {
    CHECK(calculate_accessor_offset({4}, TensorDims{{13}}) == 4);
    CHECK(calculate_accessor_offset({0, 0}, TensorDims{{5, 6}}) == 0);
    CHECK(calculate_accessor_offset({1, 0}, TensorDims{{5, 6}}) == 6);
    CHECK(calculate_accessor_offset({0, 1}, TensorDims{{5, 6}}) == 1);
    CHECK(calculate_accessor_offset({2, 4}, TensorDims{{5, 6}}) == 2 * 6 + 4);
    CHECK(calculate_accessor_offset({}, TensorDims{{}}) == 0);
    CHECK_THROWS(calculate_accessor_offset({1, 2, 4}, TensorDims{{5, 6}}));
    CHECK_THROWS(calculate_accessor_offset({2, 6}, TensorDims{{5, 6}}));
  });
  run("LocalCPUAllocator and accessors", [] {
    Allocator cpu = create_local_cpu_memory_allocator();
    CHECK(cpu.get_allocation_device_type() == DeviceType::CPU);
    GenericTensorAccessorW a = cpu.allocate_tensor(shape({2, 3}, DataType::FLOAT));
    fill_with_zeros(a);
    a.at<float>({1, 2}) = 12.0f;
    GenericTensorAccessorR r = read_only_accessor_from_write_accessor(a);
    CHECK(r.at<float>({1, 2}) == 12.0f);
    CHECK(r.get_float_ptr()[5] == 12.0f);
    CHECK_THROWS(r.get_int32_ptr());
    CHECK_THROWS(r.at<double>({0, 0}));
    GenericTensorAccessorW b = copy_tensor_accessor_w(a, cpu);
    CHECK(b.at<float>({1, 2}) == 12.0f && b.at<float>({0, 0}) == 0.0f);
    cpu.deallocate_tensor(b);
    CHECK_THROWS(cpu.deallocate_tensor(b));  // double free is an error
    CHECK(size_of_datatype(DataType::BF16) == 2 && size_of_datatype(DataType::DOUBLE) == 8);
  });
  run("CPU device type is not executed", [] {
    Allocator cpu = create_local_cpu_memory_allocator();
    LinearAttrs attrs{2, false, DataType::FLOAT, std::nullopt, std::nullopt};
    GenericTensorAccessorW x = cpu.allocate_tensor(shape({4, 3}, DataType::FLOAT));
    GenericTensorAccessorW w = cpu.allocate_tensor(shape({2, 3}, DataType::FLOAT));
    GenericTensorAccessorW y = cpu.allocate_tensor(shape({4, 2}, DataType::FLOAT));
    CHECK(!linear_init_kernel(DeviceType::CPU, device_handle_t::for_cpu(), std::nullopt, std::nullopt, false,
                              DataType::FLOAT, DataType::FLOAT, DataType::FLOAT, 4, 2)
               .has_value());
    CHECK_THROWS(linear_forward_kernel(get_cpu_device_stream(), std::nullopt, attrs, x, y, w, std::nullopt));
  });
  run("ComputationGraphBuilder: shape inference, weight layers, errors", [] {
    ComputationGraphBuilder cgb;
    tensor_guid_t ids = cgb.create_input(shape({4, 16}, DataType::INT32), CreateGrad::NO);
    tensor_guid_t emb = cgb.embedding(ids, 1000, 64, std::nullopt, DataType::BF16);
    CHECK(cgb.get_shape(emb) == shape({4, 16, 64}, DataType::BF16));
    CHECK(cgb.get_shape(cgb.get_weights_of(emb).at(0)) == shape({1000, 64}, DataType::FLOAT));
    tensor_guid_t bag = cgb.embedding(ids, 1000, 64, AggregateOp::SUM);
    CHECK(cgb.get_shape(bag) == shape({4, 64}, DataType::FLOAT));  // embedding.cc:31-36
    tensor_guid_t att = cgb.multihead_attention(emb, emb, emb, 64, 1, 64, 64, 0.0f, false);
    CHECK(cgb.get_shape(att) == shape({4, 16, 64}, DataType::BF16));
    // q, k, v projections [64 x 64] and the output projection (attention.cc:165-185)
    CHECK(get_num_elements(cgb.get_shape(cgb.get_weights_of(att).at(0)).dims) == 4 * 64 * 64);
    tensor_guid_t ln = cgb.layer_norm(cgb.add(att, emb), {-1}, true, 1e-5f);
    CHECK(cgb.get_weights_of(ln).size() == 2 && cgb.get_shape(cgb.get_weights_of(ln)[0]) == shape({64}, DataType::BF16));
    tensor_guid_t fc = cgb.dense(ln, 96, Activation::RELU, true);
    CHECK(cgb.get_shape(fc) == shape({4, 16, 96}, DataType::BF16));
    CHECK(cgb.get_shape(cgb.get_weights_of(fc).at(0)) == shape({96, 64}, DataType::BF16));
    CHECK(cgb.get_shape(cgb.get_weights_of(fc).at(1)) == shape({96}, DataType::BF16));
    CHECK(cgb.get_shape(cgb.softmax(cgb.cast(fc, DataType::FLOAT))) == shape({4, 16, 96}, DataType::FLOAT));
    CHECK(cgb.get_weights_of(cgb.dropout(fc, 0.1f)).empty());
    // GELU after a dense layer is a layer of its own (Linear's backward has no GELU)
    tensor_guid_t ge = cgb.dense(ln, 96, Activation::GELU, true);
    CHECK(std::holds_alternative<ElementUnaryAttrs>(cgb.computation_graph.layers[cgb.computation_graph.tensors[ge.raw].source.raw].attrs.op_attrs));
    CHECK_THROWS(cgb.add(fc, ln));                                   // 96 vs 64 wide: sizes do not divide
    CHECK_THROWS(cgb.layer_norm(fc, {0}, true, 1e-5f));              // a leading axis
    CHECK_THROWS(cgb.embedding(fc, 10, 4, std::nullopt));            // float indices
    CHECK_THROWS(cgb.multihead_attention(fc, ln, ln, 64, 1, 64, 64, 0.0f, false, true));  // add_bias_kv
    CHECK_THROWS(add_layer(cgb.computation_graph,
                           LayerAttrs{LinearAttrs{8, false, DataType::BF16, std::nullopt, std::nullopt}, std::nullopt}, {ln},
                           {cgb.get_weights_of(fc).at(0)}));         // a weight of the wrong shape
    ComputationGraph const &cg = cgb.computation_graph;
    CHECK(topological_ordering(cg).size() == cg.layers.size());
    bool producers_first = true;
    for (size_t l = 0; l < cg.layers.size(); l++) {
      for (tensor_guid_t t : cg.layers[l].inputs) producers_first = producers_first && cg.tensors[t.raw].source.raw < (int)l;
      for (tensor_guid_t t : cg.layers[l].weights) producers_first = producers_first && cg.tensors[t.raw].source.raw < (int)l;
    }
    CHECK(producers_first);
  });

  run("get_optimizer_attrs_for_next_iter (lib/pcg/src/pcg/optimizer_attrs.cc:6-26)", [] {
    OptimizerAttrs sgd = SGDOptimizerAttrs{0.1, 0.9, true, 0.0};
    CHECK(std::get<SGDOptimizerAttrs>(get_optimizer_attrs_for_next_iter(sgd)).lr == 0.1);
    AdamOptimizerAttrs a{1e-3, 0.9, 0.999, 0.0, 1e-3, 1.0, 1.0, 1e-8};
    for (int t = 1; t <= 3; t++) {
      a = std::get<AdamOptimizerAttrs>(get_optimizer_attrs_for_next_iter(OptimizerAttrs{a}));
      CHECK(std::fabs(a.beta_t - std::pow(0.9, t)) < 1e-12 && std::fabs(a.beta2_t - std::pow(0.999, t)) < 1e-12);
      CHECK(std::fabs(a.alpha_t - 1e-3 * std::sqrt(1 - std::pow(0.999, t)) / (1 - std::pow(0.9, t))) < 1e-12);
    }
    CHECK(get_loss_function(LossAttrs{SparseCategoricalCrossEntropyLossAttrs{false}}) == LossFunction::SPARSE_CATEGORICAL_CROSSENTROPY);
    CHECK(get_loss_function(LossAttrs{NonconfigurableLossAttrs{LossFunction::IDENTITY}}) == LossFunction::IDENTITY);
  });
}

// ---------------------------------------------------------------------------
static void gpu_tests() {
  ManagedPerDeviceFFHandle managed_handle = initialize_single_gpu_handle(1024 * 1024, true);
  device_handle_t handle = device_handle_t_from_managed_ff_handle(managed_handle);
  device_stream_t stream = get_gpu_device_stream();
  Allocator gpu = create_local_cuda_memory_allocator();

  run("A translation unit with the reference's include lines and get<DataType>() / at<DataType>() accessor calls", [&] {
    std::string const bad = reference_style_translation_unit();
    if (!bad.empty()) printf("  failed: %s\n", bad.c_str());
    CHECK(bad.empty());
  });

  run("linear_forward_kernel / linear_backward_kernel (reference KAT, exact)", [&] {
    std::vector<float> x = {3, 3, 6, 2, 1, 5, 1, 2, -2, 8, 0.5, -3}, w = {1, 2, 1.5, 0.5, 4, -1}, b = {3, -1};
    std::vector<float> dy = {1, -0.5, 2, -2, 1, 9, -3.5, 1};
    LinearAttrs attrs{2, true, DataType::FLOAT, std::nullopt, std::nullopt};
    auto state = linear_init_kernel(DeviceType::GPU, handle, std::nullopt, std::nullopt, true, DataType::FLOAT,
                                    DataType::FLOAT, DataType::FLOAT, 4, 2);
    auto X = device_accessor(gpu, shape({4, 3}, DataType::FLOAT), x);
    auto W = device_accessor(gpu, shape({2, 3}, DataType::FLOAT), w);
    auto B = device_accessor(gpu, shape({2}, DataType::FLOAT), b);
    auto Y = gpu.allocate_tensor(shape({4, 2}, DataType::FLOAT));
    linear_forward_kernel(stream, state, attrs, X, Y, W, GenericTensorAccessorR(B));
    CHECK(to_host(Y) == (std::vector<float>{21, 6.5, 14.5, -1, 5, 9.5, 7.5, 8}));
    auto DY = device_accessor(gpu, shape({4, 2}, DataType::FLOAT), dy);
    auto DX = gpu.allocate_tensor(X.shape);
    auto DW = gpu.allocate_tensor(W.shape);
    auto DB = gpu.allocate_tensor(B.shape);
    fill_with_zeros(DX); fill_with_zeros(DW); fill_with_zeros(DB);
    linear_backward_kernel(stream, state, attrs, Y, DY, X, DX, W, DW, DB);
    CHECK(to_host(DX) == (std::vector<float>{0.75, 0, 2, 1, -4, 5, 5.5, 38, -7.5, -3, -3, -6.25}));
    CHECK(to_host(DW) == (std::vector<float>{-20, 5.25, 24.5, 11.5, 15, -34}));
    CHECK(to_host(DB) == (std::vector<float>{0.5, 7.5}));
    // gradients accumulate on the GPU path (beta = 1)
    linear_backward_kernel(stream, state, attrs, Y, DY, X, DX, W, DW, DB);
    CHECK(to_host(DB) == (std::vector<float>{1.0, 15.0}));
    linear_cleanup_kernel(DeviceType::GPU, state);
  });

  run("linear with ReLU vs oracle (config-1 shape)", [&] {
    int batch = 32, in = 64, out = 128;
    auto x = random_vec(batch * in, 1), w = random_vec(out * in, 2, -0.05f, 0.05f), b = random_vec(out, 3, -0.05f, 0.05f);
    auto dy = random_vec(batch * out, 4);
    std::vector<float> y(batch * out), dx(batch * in), dw(out * in), db(out);
    orc_linear_forward(0, x.data(), y.data(), w.data(), b.data(), batch, in, out);
    orc_linear_backward(0, 0, y.data(), dy.data(), x.data(), dx.data(), w.data(), dw.data(), db.data(), batch, in, out);
    LinearAttrs attrs{out, true, DataType::FLOAT, Activation::RELU, std::nullopt};
    auto state = linear_init_kernel(DeviceType::GPU, handle, Activation::RELU, std::nullopt, true, DataType::FLOAT,
                                    DataType::FLOAT, DataType::FLOAT, batch, out);
    auto X = device_accessor(gpu, shape({batch, in}, DataType::FLOAT), x);
    auto W = device_accessor(gpu, shape({out, in}, DataType::FLOAT), w);
    auto B = device_accessor(gpu, shape({out}, DataType::FLOAT), b);
    auto DY = device_accessor(gpu, shape({batch, out}, DataType::FLOAT), dy);
    auto Y = gpu.allocate_tensor(shape({batch, out}, DataType::FLOAT));
    auto DX = gpu.allocate_tensor(X.shape), DW = gpu.allocate_tensor(W.shape), DB = gpu.allocate_tensor(B.shape);
    fill_with_zeros(DX); fill_with_zeros(DW); fill_with_zeros(DB);
    auto ms = profiling_wrapper(linear_forward_kernel, ProfilingSettings{1, 3}, DeviceType::GPU, state, attrs,
                                GenericTensorAccessorR(X), Y, GenericTensorAccessorR(W),
                                std::optional<GenericTensorAccessorR>(B));
    CHECK(ms.has_value() && ms->value > 0.0f);
    CHECK(close(to_host(Y), y, 1e-5));
    linear_backward_kernel(stream, state, attrs, Y, DY, X, DX, W, DW, DB);
    CHECK(close(to_host(DX), dx, 1e-5) && close(to_host(DW), dw, 1e-5) && close(to_host(DB), db, 1e-5));
    // {0, 0}: runs once, reports nothing
    fill_with_zeros(Y);
    auto none = profiling_wrapper(linear_forward_kernel, ProfilingSettings{0, 0}, DeviceType::GPU, state, attrs,
                                  GenericTensorAccessorR(X), Y, GenericTensorAccessorR(W),
                                  std::optional<GenericTensorAccessorR>(B));
    CHECK(!none.has_value() && contains_non_zero(to_host(Y)));
    linear_cleanup_kernel(DeviceType::GPU, state);
  });

  run("linear backward with an L2 regularizer (reference KAT + lambda W), L1 refused", [&] {
    std::vector<float> x = {3, 3, 6, 2, 1, 5, 1, 2, -2, 8, 0.5, -3}, w = {1, 2, 1.5, 0.5, 4, -1};
    std::vector<float> dy = {1, -0.5, 2, -2, 1, 9, -3.5, 1};
    float const lambda = 0.5f;
    std::optional<RegularizerAttrs> reg = RegularizerAttrs{L2RegularizerAttrs{lambda}};
    LinearAttrs attrs{2, false, DataType::FLOAT, std::nullopt, reg};
    auto state = linear_init_kernel(DeviceType::GPU, handle, std::nullopt, reg, false, DataType::FLOAT, DataType::FLOAT,
                                    DataType::FLOAT, 4, 2);
    auto X = device_accessor(gpu, shape({4, 3}, DataType::FLOAT), x);
    auto W = device_accessor(gpu, shape({2, 3}, DataType::FLOAT), w);
    auto DY = device_accessor(gpu, shape({4, 2}, DataType::FLOAT), dy);
    auto Y = gpu.allocate_tensor(shape({4, 2}, DataType::FLOAT));
    auto DX = gpu.allocate_tensor(X.shape), DW = gpu.allocate_tensor(W.shape);
    fill_with_zeros(DX); fill_with_zeros(DW);
    linear_forward_kernel(stream, state, attrs, X, Y, W, std::nullopt);
    linear_backward_kernel(stream, state, attrs, Y, DY, X, DX, W, DW, std::nullopt);
    // the known-answer weight gradient {-20, 5.25, 24.5, 11.5, 15, -34} plus 0.5 W
    CHECK(to_host(DW) == (std::vector<float>{-19.5, 6.25, 25.25, 11.75, 17, -34.5}));
    std::vector<float> want = {-20, 5.25, 24.5, 11.5, 15, -34};
    orc_linear_l2_regularizer_grad(w.data(), want.data(), 6, lambda);
    CHECK(to_host(DW) == want);
    // second call: (dW + g^T x) + lambda W again
    linear_backward_kernel(stream, state, attrs, Y, DY, X, DX, W, DW, std::nullopt);
    CHECK(to_host(DW) == (std::vector<float>{-39, 12.5, 50.5, 23.5, 34, -69}));
    linear_cleanup_kernel(DeviceType::GPU, state);
    CHECK_THROWS(linear_init_kernel(DeviceType::GPU, handle, std::nullopt, RegularizerAttrs{L1RegularizerAttrs{0.1f}}, false,
                                    DataType::FLOAT, DataType::FLOAT, DataType::FLOAT, 4, 2));
  });

  run("LayerNorm forward/backward vs oracle", [&] {
    int64_t M = 37, N = 96;
    auto x = random_vec(M * N, 5, -2, 2), g = random_vec(N, 6, 0.5f, 1.5f), b = random_vec(N, 7), dy = random_vec(M * N, 8);
    std::vector<float> y(M * N), mean(M), rstd(M), dx(M * N), dg(N), db(N);
    orc_layer_norm_forward(x.data(), y.data(), g.data(), b.data(), mean.data(), rstd.data(), M, N, 1e-5f);
    orc_layer_norm_backward(dy.data(), x.data(), mean.data(), rstd.data(), g.data(), dx.data(), dg.data(), db.data(), M, N, 0);
    auto state = Kernels::LayerNorm::init_kernel(DeviceType::GPU, handle, gpu, true, M, N, 1e-5f);
    auto X = device_accessor(gpu, shape({M, N}, DataType::FLOAT), x);
    auto G = device_accessor(gpu, shape({N}, DataType::FLOAT), g);
    auto Bt = device_accessor(gpu, shape({N}, DataType::FLOAT), b);
    auto DY = device_accessor(gpu, shape({M, N}, DataType::FLOAT), dy);
    auto Y = gpu.allocate_tensor(X.shape), DX = gpu.allocate_tensor(X.shape);
    auto DG = gpu.allocate_tensor(G.shape), DB = gpu.allocate_tensor(G.shape);
    fill_with_zeros(DX);
    Kernels::LayerNorm::forward_kernel(stream, state, X, Y, G, Bt);
    CHECK(close(to_host(Y), y, 2e-5));
    Kernels::LayerNorm::backward_kernel(stream, state, DY, X, DX, G, DG, DB);
    CHECK(close(to_host(DX), dx, 5e-5) && close(to_host(DG), dg, 5e-5) && close(to_host(DB), db, 5e-5));
    Kernels::LayerNorm::cleanup_kernel(DeviceType::GPU, state);
  });

  run("Softmax over the channel of (n,c,h,w); reference backward is a copy", [&] {
    int n = 2, c = 5, h = 3, w = 4;
    auto x = random_vec(n * c * h * w, 9, -4, 4), dy = random_vec(n * c * h * w, 10);
    std::vector<float> y(x.size()), dx(x.size());
    orc_softmax_forward(x.data(), y.data(), n, c, h * w);
    auto state = Kernels::Softmax::init_kernel(DeviceType::GPU, handle, ff_dim_t{1}, n, c, h, w);
    auto X = device_accessor(gpu, shape({n, c, h, w}, DataType::FLOAT), x);
    auto DY = device_accessor(gpu, X.shape, dy);
    auto Y = gpu.allocate_tensor(X.shape), DX = gpu.allocate_tensor(X.shape);
    Kernels::Softmax::forward_kernel(stream, state, X.get_float_ptr(), Y.get_float_ptr());
    CHECK(close(to_host(Y), y, 2e-5));
    Kernels::Softmax::backward_kernel(stream, DY.get_float_ptr(), DX.get_float_ptr(), x.size());
    CHECK(to_host(DX) == dy);
    orc_softmax_backward(to_host(Y).data(), dy.data(), dx.data(), n, c, h * w);
    Kernels::Softmax::backward_kernel(stream, state, Y, DY, DX);
    CHECK(close(to_host(DX), dx, 5e-5));
  });

  run("Dropout mask equals the oracle's stream bit for bit", [&] {
    size_t n = 10 * 1000 + 3;
    auto x = random_vec(n, 11);
    std::vector<float> y(n), dx(n);
    orc_dropout_forward(x.data(), y.data(), n, 0.1f, 12345ull, 0);
    orc_dropout_backward(x.data(), dx.data(), n, 0.1f, 12345ull, 0, 0);
    TensorShape s = shape({(int64_t)n}, DataType::FLOAT);
    auto state = Kernels::Dropout::init_kernel(DeviceType::GPU, handle, 0.1f, 12345ull, s, gpu);
    auto X = device_accessor(gpu, s, x);
    auto Y = gpu.allocate_tensor(s), DX = gpu.allocate_tensor(s);
    Kernels::Dropout::forward_kernel(stream, state, X.get_float_ptr(), Y.get_float_ptr());
    CHECK(to_host(Y) == y);
    CHECK(contains_non_zero(to_host(Y)));
    Kernels::Dropout::backward_kernel(stream, state, X.get_float_ptr(), DX.get_float_ptr());
    CHECK(to_host(DX) == dx);
  });

  run("ElementUnary GELU and ElementBinary add/mul vs oracle", [&] {
    size_t n = 5000;
    auto x = random_vec(n, 12, -3, 3), r = random_vec(n, 13, 0.5f, 2.0f), dy = random_vec(n, 14);
    TensorShape s = shape({50, 100}, DataType::FLOAT);
    ElementUnaryAttrs gelu{OperatorType::GELU, std::nullopt};
    auto ustate = Kernels::ElementUnary::init_kernel(DeviceType::GPU, s, s, gelu);
    std::vector<float> y(n), dx(n, 0.0f);
    orc_element_unary_forward(67, 0.0f, x.data(), y.data(), n);
    orc_element_unary_backward(67, 0.0f, y.data(), dy.data(), x.data(), dx.data(), n, -1);
    auto X = device_accessor(gpu, s, x), R = device_accessor(gpu, s, r), DY = device_accessor(gpu, s, dy);
    auto Y = gpu.allocate_tensor(s), DX = gpu.allocate_tensor(s), DR = gpu.allocate_tensor(s);
    fill_with_zeros(DX);
    Kernels::ElementUnary::forward_kernel(stream, ustate, gelu, handle, X, Y);
    CHECK(close(to_host(Y), y, 2e-5));
    Kernels::ElementUnary::backward_kernel(stream, ustate, gelu, handle, Y, DY, X, DX);
    CHECK(close(to_host(DX), dx, 2e-5));
    for (OperatorType op : {OperatorType::EW_ADD, OperatorType::EW_MUL}) {
      auto bstate = Kernels::ElementBinary::init_kernel(DeviceType::GPU, handle, op, false, false, s, s, s);
      std::vector<float> o(n), dl(n, 0.0f), dr(n, 0.0f);
      orc_element_binary_forward(static_cast<int>(op), x.data(), r.data(), o.data(), n, n, n);
      orc_element_binary_backward(static_cast<int>(op), dy.data(), x.data(), r.data(), dl.data(), dr.data(), n, 1);
      Kernels::ElementBinary::forward_kernel(stream, bstate, X.get_float_ptr(), R.get_float_ptr(), Y.get_float_ptr(),
                                             op, false, handle);
      CHECK(close(to_host(Y), o, 1e-6));
      fill_with_zeros(DX); fill_with_zeros(DR);
      Kernels::ElementBinary::backward_kernel(stream, bstate, DY.get_float_ptr(), X.get_float_ptr(), R.get_float_ptr(),
                                              DX.get_float_ptr(), DR.get_float_ptr(), op, false, false, handle);
      CHECK(close(to_host(DX), dl, 1e-6) && close(to_host(DR), dr, 1e-6));
    }
  });

  run("ElementBinary with a broadcast operand: its gradient is the reduction the reference asks cuDNN for", [&] {
    // element_binary_kernels.cu:268-396 (broadcast_inputRHS): add reduces dy, mul reduces dy * lhs
    int64_t rows = 50, cols = 100;
    size_t n = rows * cols;
    auto x = random_vec(n, 31, -2, 2), b = random_vec(cols, 32, 0.5f, 2.0f), dy = random_vec(n, 33);
    TensorShape s = shape({rows, cols}, DataType::FLOAT), sb = shape({cols}, DataType::FLOAT);
    auto X = device_accessor(gpu, s, x), B = device_accessor(gpu, sb, b), DY = device_accessor(gpu, s, dy);
    auto Y = gpu.allocate_tensor(s), DX = gpu.allocate_tensor(s), DB = gpu.allocate_tensor(sb);
    for (OperatorType op : {OperatorType::EW_ADD, OperatorType::EW_MUL}) {
      bool const mul = op == OperatorType::EW_MUL;
      auto bstate = Kernels::ElementBinary::init_kernel(DeviceType::GPU, handle, op, false, true, s, sb, s);
      std::vector<float> o(n), dl(n), dr(cols);
      for (int64_t j = 0; j < cols; j++) {
        double acc = 0.0;
        for (int64_t i = 0; i < rows; i++) {
          size_t k = i * cols + j;
          o[k] = mul ? x[k] * b[j] : x[k] + b[j];
          dl[k] = mul ? dy[k] * b[j] : dy[k];
          acc += mul ? (double)dy[k] * x[k] : (double)dy[k];
        }
        dr[j] = (float)acc;
      }
      Kernels::ElementBinary::forward_kernel(stream, bstate, X.get_float_ptr(), B.get_float_ptr(), Y.get_float_ptr(),
                                             op, false, handle);
      CHECK(close(to_host(Y), o, 1e-6));
      fill_with_zeros(DX); fill_with_zeros(DB);
      Kernels::ElementBinary::backward_kernel(stream, bstate, DY.get_float_ptr(), X.get_float_ptr(), B.get_float_ptr(),
                                              DX.get_float_ptr(), DB.get_float_ptr(), op, false, true, handle);
      CHECK(close(to_host(DX), dl, 1e-6));
      CHECK(close(to_host(DB), dr, 1e-5));
      // a second call adds (the reference's beta = 1)
      Kernels::ElementBinary::backward_kernel(stream, bstate, DY.get_float_ptr(), X.get_float_ptr(), B.get_float_ptr(),
                                              nullptr, DB.get_float_ptr(), op, false, true, handle);
      for (auto &v : dr) v *= 2.0f;
      CHECK(close(to_host(DB), dr, 1e-5));
    }
    // leading 1s are the same pattern; a size-1 dim in the middle or at the end is another one
    // (the kernels would repeat the operand over the wrong elements) and is refused
    TensorShape out3 = shape({4, 5, 6}, DataType::FLOAT);
    CHECK(Kernels::ElementBinary::init_kernel(DeviceType::GPU, handle, OperatorType::EW_ADD, false, true, out3,
                                              shape({1, 1, 6}, DataType::FLOAT), out3).has_value());
    CHECK(Kernels::ElementBinary::init_kernel(DeviceType::GPU, handle, OperatorType::EW_ADD, false, true, out3,
                                              shape({5, 6}, DataType::FLOAT), out3).has_value());
    CHECK_THROWS(Kernels::ElementBinary::init_kernel(DeviceType::GPU, handle, OperatorType::EW_ADD, true, false,
                                                     shape({4, 1, 6}, DataType::FLOAT), out3, out3));
    CHECK_THROWS(Kernels::ElementBinary::init_kernel(DeviceType::GPU, handle, OperatorType::EW_MUL, false, true, out3,
                                                     shape({4, 5, 1}, DataType::FLOAT), out3));
    {
      ComputationGraphBuilder bld;
      tensor_guid_t a = bld.create_input(out3, CreateGrad::YES), c = bld.create_input(shape({4, 1, 6}, DataType::FLOAT), CreateGrad::YES);
      CHECK_THROWS(bld.add(a, c));
    }
  });

  run("Embedding gather (exact) and scatter-add vs oracle", [&] {
    int64_t V = 97, D = 32, B = 40, bag = 4;
    auto w = random_vec(V * D, 15), dy = random_vec(B * D, 16);
    std::vector<int64_t> idx(B * bag);
    std::mt19937 gen(0);
    for (auto &i : idx) i = gen() % V;
    std::vector<int32_t> idx32(idx.begin(), idx.end());
    std::vector<float> out(B * D), dw(V * D, 0.0f);
    orc_embedding_forward(idx.data(), out.data(), w.data(), 0, B, bag, D, V);
    orc_embedding_backward_f64(idx.data(), dy.data(), dw.data(), 0, B, bag, D, V);
    Allocator cpu = create_local_cpu_memory_allocator();
    GenericTensorAccessorW hidx = cpu.allocate_tensor(shape({B, bag}, DataType::INT32));
    memcpy(hidx.ptr, idx32.data(), idx32.size() * 4);
    GenericTensorAccessorW I = copy_tensor_accessor_w(hidx, gpu);
    auto W = device_accessor(gpu, shape({V, D}, DataType::FLOAT), w);
    auto DYa = device_accessor(gpu, shape({B, D}, DataType::FLOAT), dy);
    auto O = gpu.allocate_tensor(shape({B, D}, DataType::FLOAT)), DW = gpu.allocate_tensor(W.shape);
    fill_with_zeros(DW);
    Kernels::Embedding::forward_kernel(stream, I, O, W, DataType::INT32, DataType::FLOAT, AggregateOp::SUM, 2, 2, (int)B);
    CHECK(to_host(O) == out);
    Kernels::Embedding::backward_kernel(stream, DYa, I, DW, DataType::FLOAT, DataType::INT32, AggregateOp::SUM, 2, 2, (int)B);
    CHECK(close(to_host(DW), dw, 1e-5));
    // DOUBLE tables (the reference instantiates HALF, FLOAT and DOUBLE): one type throughout.  The
    // values are quarters of small integers, so every sum is exact in fp32 as in double and the
    // fp32 oracle's result, widened, is the expected one to the bit.
    std::vector<double> wd(V * D), dyd(B * D);
    std::vector<float> wq(V * D), dyq(B * D), outq(B * D), dwq(V * D, 0.0f);
    for (size_t i = 0; i < wd.size(); i++) wd[i] = wq[i] = (float)((int)(gen() % 65) - 32) / 4.0f;
    for (size_t i = 0; i < dyd.size(); i++) dyd[i] = dyq[i] = (float)((int)(gen() % 33) - 16) / 4.0f;
    orc_embedding_forward(idx.data(), outq.data(), wq.data(), 0, B, bag, D, V);
    orc_embedding_backward(idx.data(), dyq.data(), dwq.data(), 0, B, bag, D, V);
    GenericTensorAccessorW hw = cpu.allocate_tensor(shape({V, D}, DataType::DOUBLE)), hdy = cpu.allocate_tensor(shape({B, D}, DataType::DOUBLE));
    memcpy(hw.ptr, wd.data(), wd.size() * 8);
    memcpy(hdy.ptr, dyd.data(), dyd.size() * 8);
    GenericTensorAccessorW Wd = copy_tensor_accessor_w(hw, gpu), DYd = copy_tensor_accessor_w(hdy, gpu);
    auto Od = gpu.allocate_tensor(shape({B, D}, DataType::DOUBLE)), DWd = gpu.allocate_tensor(Wd.shape);
    fill_with_zeros(DWd);
    Kernels::Embedding::forward_kernel(stream, I, Od, Wd, DataType::INT32, DataType::DOUBLE, AggregateOp::SUM, 2, 2, (int)B);
    Kernels::Embedding::backward_kernel(stream, DYd, I, DWd, DataType::DOUBLE, DataType::INT32, AggregateOp::SUM, 2, 2, (int)B);
    GenericTensorAccessorW hod = copy_tensor_accessor_w(Od, cpu), hdwd = copy_tensor_accessor_w(DWd, cpu);
    bool same = true;
    for (int64_t i = 0; i < B * D; i++) same = same && hod.get<DataType::DOUBLE>()[i] == (double)outq[i];
    for (int64_t i = 0; i < V * D; i++) same = same && hdwd.get<DataType::DOUBLE>()[i] == (double)dwq[i];
    CHECK(same);
    // a FLOAT gradient into a DOUBLE weight_grad is refused
    CHECK_THROWS(Kernels::Embedding::backward_kernel(stream, DYa, I, DWd, DataType::FLOAT, DataType::INT32, AggregateOp::SUM, 2, 2, (int)B));
  });

  run("MultiHeadAttention (bf16 accessors) vs oracle", [&] {
    int B = 2, H = 4, E = 64, D = 64, S = 20;  // the reference test's sizes, [batch, seq, size]
    auto q = random_vec(B * S * E, 17), dout = random_vec(B * S * E, 18);
    size_t nw = (size_t)H * D * 3 * E + (size_t)E * H * D;
    auto w = random_vec(nw, 19, -0.2f, 0.2f);
    for (auto *v : {&q, &dout, &w}) orc_round_bf16_array(v->data(), v->size());
    orc_mha_desc_t od{B, H, E, E, E, D, D, D, E, S, S, 1.0f, 0};
    std::vector<float> out(B * S * E), dq(q.size()), dk(q.size()), dv(q.size()), dw(nw, 0.0f);
    orc_mha_forward(&od, q.data(), q.data(), q.data(), w.data(), out.data(), 1);
    orc_mha_backward(&od, q.data(), q.data(), q.data(), w.data(), dout.data(), dq.data(), dk.data(), dv.data(), dw.data(), 1);
    for (size_t i = 0; i < dq.size(); i++) dq[i] += dk[i] + dv[i];
    auto state = Kernels::MultiHeadAttention::init_kernel(DeviceType::GPU, handle, gpu, B, H, E, E, E, D, D, D, E, S, S,
                                                          false, DataType::BF16, 1.0f, false);
    CHECK(state->weightSize == nw * 2);
    auto Q = device_accessor(gpu, shape({B, S, E}, DataType::BF16), q);
    auto W = device_accessor(gpu, shape({(int64_t)nw}, DataType::BF16), w);
    auto DO = device_accessor(gpu, Q.shape, dout);
    auto O = gpu.allocate_tensor(Q.shape), DQ = gpu.allocate_tensor(Q.shape), DW = gpu.allocate_tensor(W.shape);
    fill_with_zeros(DQ); fill_with_zeros(DW);
    Kernels::MultiHeadAttention::forward_kernel(stream, state, Q, Q, Q, W, O);
    CHECK(contains_non_zero(to_host(O)));
    CHECK(close(to_host(O), out, 2e-2));
    Kernels::MultiHeadAttention::backward_kernel(stream, state, Q, DQ, Q, std::nullopt, Q, std::nullopt, W, DW, DO);
    CHECK(close(to_host(DQ), dq, 2e-2) && close(to_host(DW), dw, 2e-2));
    Kernels::MultiHeadAttention::cleanup_kernel(DeviceType::GPU, gpu, state);
    // float pointers belong to a FLOAT state
    CHECK_THROWS(Kernels::MultiHeadAttention::forward_kernel(stream, state, (float const *)Q.ptr, (float const *)Q.ptr,
                                                             (float const *)Q.ptr, (float const *)W.ptr, (float *)O.ptr));
  });
  run("MultiHeadAttention, the reference's float signature (fp32, scale 1, q = k = v, NULL dk/dv) vs oracle", [&] {
    // the sizes of lib/kernels/test/src/test_attention_kernel.cc, [batch, seq, size]
    int B = 2, H = 4, E = 64, D = 64, S = 20;
    auto q = random_vec(B * S * E, 27, -0.5f, 0.5f), dout = random_vec(B * S * E, 28);
    size_t nw = (size_t)H * D * 3 * E + (size_t)E * H * D;
    auto w = random_vec(nw, 29, -0.2f, 0.2f);
    orc_mha_desc_t od{B, H, E, E, E, D, D, D, E, S, S, 1.0f, 0};
    std::vector<float> out(B * S * E), dq(q.size()), dk(q.size()), dv(q.size()), dw(nw, 0.0f);
    orc_mha_forward(&od, q.data(), q.data(), q.data(), w.data(), out.data(), 0);
    orc_mha_backward(&od, q.data(), q.data(), q.data(), w.data(), dout.data(), dq.data(), dk.data(), dv.data(), dw.data(), 0);
    for (size_t i = 0; i < dq.size(); i++) dq[i] += dk[i] + dv[i];
    auto state = Kernels::MultiHeadAttention::init_kernel(DeviceType::GPU, handle, gpu, B, H, E, E, E, D, D, D, E, S, S, false);
    CHECK(state->weightSize == nw * 4);
    auto Q = device_accessor(gpu, shape({B, S, E}, DataType::FLOAT), q);
    auto W = device_accessor(gpu, shape({(int64_t)nw}, DataType::FLOAT), w);
    auto DO = device_accessor(gpu, Q.shape, dout);
    auto O = gpu.allocate_tensor(Q.shape), DW = gpu.allocate_tensor(W.shape);
    // the input gradient is stored, not added to: start it from values that would show
    auto DQ = device_accessor(gpu, Q.shape, random_vec(q.size(), 30, 5.0f, 6.0f));
    fill_with_zeros(DW);
    Kernels::MultiHeadAttention::forward_kernel(stream, state, Q.get_float_ptr(), Q.get_float_ptr(), Q.get_float_ptr(),
                                                W.get_float_ptr(), O.get_float_ptr());
    CHECK(contains_non_zero(to_host(O)));
    CHECK(close(to_host(O), out, 1e-5));
    Kernels::MultiHeadAttention::backward_kernel(stream, state, Q.get_float_ptr(), DQ.get_float_ptr(), Q.get_float_ptr(),
                                                 nullptr, Q.get_float_ptr(), nullptr, W.get_float_ptr(), DW.get_float_ptr(),
                                                 DO.get_float_ptr());
    CHECK(close(to_host(DQ), dq, 1e-5));
    CHECK(close(to_host(DW), dw, 1e-5));
    // the weight gradient is added to (CUDNN_WGRAD_MODE_ADD): a second call doubles it
    Kernels::MultiHeadAttention::backward_kernel(stream, state, Q.get_float_ptr(), DQ.get_float_ptr(), Q.get_float_ptr(),
                                                 nullptr, Q.get_float_ptr(), nullptr, W.get_float_ptr(), DW.get_float_ptr(),
                                                 DO.get_float_ptr());
    for (auto &x : dw) x *= 2.0f;
    CHECK(close(to_host(DQ), dq, 1e-5));
    CHECK(close(to_host(DW), dw, 1e-5));
    Kernels::MultiHeadAttention::cleanup_kernel(DeviceType::GPU, gpu, state);
  });
  run("sgd_update_task / adam_update_task equal the oracle bit for bit", [&] {
    int64_t n = 10007;
    auto w = random_vec(n, 20), g = random_vec(n, 21), v = random_vec(n, 22, 0.0f, 1.0f), m = random_vec(n, 23);
    TensorShape s = shape({n}, DataType::FLOAT);
    auto W = device_accessor(gpu, s, w), G = device_accessor(gpu, s, g), V = device_accessor(gpu, s, v);
    std::vector<float> w1 = w, v1 = v;
    orc_sgd_update(0.01f, 0.9f, 1, 1e-4f, g.data(), n, 1, w1.data(), v1.data());
    sgd_update_task(stream, handle, 0.01f, 0.9f, true, 1e-4f, read_only_accessor_from_write_accessor(G), 1, W, V);
    CHECK(to_host(W) == w1 && to_host(V) == v1);
    CHECK_THROWS(sgd_update_task(stream, handle, 0.01f, 0.9f, true, 1e-4f, read_only_accessor_from_write_accessor(G), 1,
                                 W, std::nullopt));
    // a fresh second moment: the SGD velocity above may be negative
    auto M = device_accessor(gpu, s, m);
    V = device_accessor(gpu, s, v);
    std::vector<float> w2 = w1, v2 = v, m2 = m;
    orc_adam_update(1e-3f, 0.9f, 0.999f, 1e-2f, 1e-8f, g.data(), n, 1, w2.data(), v2.data(), m2.data());
    adam_update_task(stream, handle, 1e-3f, 0.9f, 0.999f, 1e-2f, 1e-8f, G.get_float_ptr(), (size_t)n, 1,
                     W.get_float_ptr(), V.get_float_ptr(), M.get_float_ptr());
    CHECK(to_host(W) == w2 && to_host(V) == v2 && to_host(M) == m2);
  });

  run("loss backward kernels equal the oracle bit for bit", [&] {
    int samples = 33, classes = 17;
    int64_t n = (int64_t)samples * classes;
    auto logit = random_vec(n, 24, 0.0f, 1.0f), label = random_vec(n, 25, 0.0f, 1.0f);
    std::vector<int> sparse(samples);
    std::mt19937 gen(1);
    for (auto &l : sparse) l = (int)(gen() % classes);
    TensorShape s = shape({samples, classes}, DataType::FLOAT);
    auto L = device_accessor(gpu, s, logit), T = device_accessor(gpu, s, label);
    auto DL = gpu.allocate_tensor(s);
    Allocator cpu = create_local_cpu_memory_allocator();
    GenericTensorAccessorW hl = cpu.allocate_tensor(shape({samples}, DataType::INT32));
    memcpy(hl.ptr, sparse.data(), sparse.size() * 4);
    GenericTensorAccessorW SL = copy_tensor_accessor_w(hl, gpu);
    float scale = 1.0f / samples;
    std::vector<float> want(n);
    orc_sparse_cce_loss_backward(want.data(), logit.data(), sparse.data(), n, samples, classes, 1, scale);
    sparse_categorical_crossentropy_loss_backward_kernel(stream, DL.get_float_ptr(), L.get_float_ptr(),
                                                         static_cast<int const *>(SL.ptr), n, n, samples, classes, 1,
                                                         scale);
    CHECK(to_host(DL) == want);
    orc_difference_loss_backward(want.data(), logit.data(), label.data(), n, scale);
    categorical_crossentropy_loss_backward_kernel(stream, DL, read_only_accessor_from_write_accessor(L),
                                                  read_only_accessor_from_write_accessor(T), scale);
    CHECK(to_host(DL) == want);
    mean_squared_error_avg_loss_backward_kernel(stream, DL.get_float_ptr(), L.get_float_ptr(), T.get_float_ptr(), n, n,
                                                scale);
    CHECK(to_host(DL) == want);
    orc_identity_loss_backward(want.data(), n, scale);
    identity_loss_backward_kernel(stream, DL.get_float_ptr(), L.get_float_ptr(), n, n, scale);
    CHECK(to_host(DL) == want);
  });

  run("Cast float -> bf16 -> float rounds to nearest even; backward accumulates", [&] {
    int64_t n = 4099;
    auto x = random_vec(n, 26, -100.0f, 100.0f);
    auto X = device_accessor(gpu, shape({n}, DataType::FLOAT), x);
    auto Y = gpu.allocate_tensor(shape({n}, DataType::BF16));
    Kernels::Cast::forward_kernel(stream, read_only_accessor_from_write_accessor(X), Y);
    std::vector<float> want = x;
    orc_round_bf16_array(want.data(), want.size());
    CHECK(to_host(Y) == want);
    auto DX = device_accessor(gpu, shape({n}, DataType::FLOAT), x);
    Kernels::Cast::backward_kernel(stream, read_only_accessor_from_write_accessor(Y), DX);
    for (int64_t i = 0; i < n; i++) want[i] += x[i];
    CHECK(to_host(DX) == want);
  });
  // lib/local-execution/test/src/local-execution/computation_graph_instance.cc:33-189
  // (CUDA twin :192-355): the same graph, loss, optimizer and assertion, and the
  // same five steps replayed with the CPU oracle.
  run("LocalBackend e2e Training: 2-layer MLP, categorical CE, SGD with momentum, 5 steps", [&] {
    int64_t batch = 10, data_dim = 16, hidden_dim = 32, output_dim = 1;
    ComputationGraph cg = make_empty_computation_graph();
    tensor_guid_t t_input = add_input_layer(cg, shape({batch, data_dim}, DataType::FLOAT)).outputs.at(0);
    tensor_guid_t t_w1 = add_weight_layer(cg, shape({hidden_dim, data_dim}, DataType::FLOAT)).outputs.at(0);
    tensor_guid_t t_w2 = add_weight_layer(cg, shape({output_dim, hidden_dim}, DataType::FLOAT)).outputs.at(0);
    tensor_guid_t t_l1 = add_layer(cg, LayerAttrs{LinearAttrs{(int)hidden_dim, false, DataType::FLOAT, Activation::RELU, std::nullopt}, std::nullopt},
                                   {t_input}, {t_w1}).outputs.at(0);
    tensor_guid_t t_l2 = add_layer(cg, LayerAttrs{LinearAttrs{(int)output_dim, false, DataType::FLOAT, Activation::RELU, std::nullopt}, std::nullopt},
                                   {t_l1}, {t_w2}).outputs.at(0);
    auto x = random_vec(batch * data_dim, 30), w1 = random_vec(hidden_dim * data_dim, 31, -0.3f, 0.5f),
         w2 = random_vec(output_dim * hidden_dim, 32, 0.0f, 0.5f);
    std::vector<float> label(batch * output_dim, 0.0f);
    auto LABEL = device_accessor(gpu, shape({batch, output_dim}, DataType::FLOAT), label);
    OptimizerAttrs optimizer = SGDOptimizerAttrs{0.001, 0.9, false, 0.001};
    device_id_t device_idx = make_device_id_t_from_idx(0, DeviceType::GPU);
    ComputationGraphInstance instance = create_computation_graph_instance(
        cg, optimizer, LossConfig{NonconfigurableLossAttrs{LossFunction::CATEGORICAL_CROSSENTROPY}, LABEL, t_l2}, {}, gpu,
        ProfilingSettings{0, 0}, handle, device_idx);
    Allocator cpu = create_local_cpu_memory_allocator();
    auto put = [&](tensor_guid_t t, std::vector<float> const &v) {
      GenericTensorAccessorW h = cpu.allocate_tensor(instance.get_tensor_accessor(t).shape);
      memcpy(h.ptr, v.data(), v.size() * 4);
      copy_accessor_data_to_l_from_r(instance.get_tensor_accessor(t), h);
    };
    put(t_input, x); put(t_w1, w1); put(t_w2, w2);

    std::vector<float> v1(w1.size(), 0.0f), v2(w2.size(), 0.0f), h(batch * hidden_dim), y(batch), dlogit(batch),
        dh(h.size()), dw1(w1.size()), dw2(w2.size()), first, last;
    for (int step = 0; step < 5; step++) {
      perform_all_passes_for_computation_graph_instance(instance, ProfilingSettings{0, 0}, handle, device_idx);
      std::vector<float> got = to_host(GenericTensorAccessorW{instance.get_loss_tensor_accessor()->shape,
                                                              const_cast<void *>(instance.get_loss_tensor_accessor()->ptr), DeviceType::GPU});
      if (step == 0) first = got;
      last = got;
      orc_linear_forward(0, x.data(), h.data(), w1.data(), nullptr, batch, data_dim, hidden_dim);
      orc_linear_forward(0, h.data(), y.data(), w2.data(), nullptr, batch, hidden_dim, output_dim);
      orc_difference_loss_backward(dlogit.data(), y.data(), label.data(), batch, 1.0f / batch);
      CHECK(close(got, dlogit, 1e-5));
      orc_linear_backward(0, 0, y.data(), dlogit.data(), h.data(), dh.data(), w2.data(), dw2.data(), nullptr, batch, hidden_dim, output_dim);
      orc_linear_backward(0, 0, h.data(), dh.data(), x.data(), nullptr, w1.data(), dw1.data(), nullptr, batch, data_dim, hidden_dim);
      orc_sgd_update(0.001f, 0.9f, 0, 0.001f, dw1.data(), (int64_t)w1.size(), 1, w1.data(), v1.data());
      orc_sgd_update(0.001f, 0.9f, 0, 0.001f, dw2.data(), (int64_t)w2.size(), 1, w2.data(), v2.data());
    }
    CHECK(contains_non_zero(first));
    CHECK(close(to_host(instance.get_tensor_accessor(t_w1)), w1, 1e-5));
    CHECK(close(to_host(instance.get_tensor_accessor(t_w2)), w2, 1e-5));
    bool did_loss_decrease = true;  // every sample's logit gradient is <= its first-step value
    for (size_t i = 0; i < first.size(); i++) did_loss_decrease = did_loss_decrease && last[i] <= first[i];
    CHECK(did_loss_decrease);
    // per-layer timings when profiling is on; FWD, LOSS, BWD, UPD all present in the order
    auto timings = perform_forward_pass_for_computation_graph_instance(instance, ProfilingSettings{1, 2}, handle, device_idx);
    CHECK(timings.size() == 2 && timings.begin()->second.has_value() && timings.begin()->second->value > 0.0f);
    int n_fwd = 0, n_bwd = 0, n_upd = 0, n_loss = 0;
    for (auto const &inv : instance.get_execution_order()) {
      n_fwd += inv.task_type == DynamicTaskType::FWD;
      n_bwd += inv.task_type == DynamicTaskType::BWD;
      n_upd += inv.task_type == DynamicTaskType::UPD;
      n_loss += inv.task_type == DynamicTaskType::LOSS;
    }
    CHECK(n_fwd == 2 && n_bwd == 2 && n_upd == 2 && n_loss == 1);
    Allocator cpu_alloc = create_local_cpu_memory_allocator();
    CHECK_THROWS(create_computation_graph_instance(cg, optimizer, std::nullopt, {}, cpu_alloc, ProfilingSettings{0, 0},
                                                   device_handle_t::for_cpu(), make_device_id_t_from_idx(0, DeviceType::CPU)));
  });

  // The reference transformer ends in dense -> softmax with a sparse categorical cross-entropy
  // on the softmax output (lib/models/src/models/transformer/transformer.cc:160-170).  The loss
  // kernel writes (p - onehot) / batch into the gradient of p, which is the cross-entropy's
  // gradient at the softmax INPUT: the softmax in front of the loss must pass it through.
  run("Step driver: Dense -> Softmax -> sparse categorical CE; the Dense output's gradient is (p - y) / batch", [&] {
    int64_t batch = 12, in_dim = 24, classes = 10;
    ComputationGraphBuilder b;
    tensor_guid_t x = b.create_input(shape({batch, in_dim}, DataType::FLOAT), CreateGrad::NO);
    tensor_guid_t z = b.dense(x, (int)classes, std::nullopt, true);
    tensor_guid_t prob = b.softmax(z);
    auto xs = random_vec(batch * in_dim, 40), w = random_vec(classes * in_dim, 41, -0.5f, 0.5f), bias = random_vec(classes, 42);
    std::vector<int> sparse(batch);
    for (int64_t i = 0; i < batch; i++) sparse[i] = (int)((i * 7 + 3) % classes);
    Allocator cpu = create_local_cpu_memory_allocator();
    GenericTensorAccessorW hl = cpu.allocate_tensor(shape({batch}, DataType::INT32));
    memcpy(hl.ptr, sparse.data(), sparse.size() * 4);
    GenericTensorAccessorW LABEL = copy_tensor_accessor_w(hl, gpu);
    OptimizerAttrs optimizer = SGDOptimizerAttrs{0.1, 0.0, false, 0.0};
    device_id_t device_idx = make_device_id_t_from_idx(0, DeviceType::GPU);
    ComputationGraphInstance instance = create_computation_graph_instance(
        b.computation_graph, optimizer, LossConfig{SparseCategoricalCrossEntropyLossAttrs{false}, LABEL, prob}, {}, gpu,
        ProfilingSettings{0, 0}, handle, device_idx);
    auto put = [&](tensor_guid_t t, std::vector<float> const &v) {
      GenericTensorAccessorW h = cpu.allocate_tensor(instance.get_tensor_accessor(t).shape);
      memcpy(h.ptr, v.data(), v.size() * 4);
      copy_accessor_data_to_l_from_r(instance.get_tensor_accessor(t), h);
    };
    std::vector<tensor_guid_t> weights = b.get_weights_of(z);
    put(x, xs); put(weights.at(0), w); put(weights.at(1), bias);
    perform_all_passes_for_computation_graph_instance(instance, ProfilingSettings{0, 0}, handle, device_idx);
    std::vector<float> zs(batch * classes), p(zs.size()), dz(zs.size()), dw(w.size()), db(bias.size());
    orc_linear_forward(-1, xs.data(), zs.data(), w.data(), bias.data(), batch, in_dim, classes);
    orc_softmax_forward(zs.data(), p.data(), batch, classes, 1);
    orc_sparse_cce_loss_backward(dz.data(), p.data(), sparse.data(), batch * classes, batch, classes, 1, 1.0f / batch);
    CHECK(close(to_host(instance.get_tensor_accessor(prob)), p, 1e-5));
    CHECK(close(to_host(*instance.get_gradient_accessor(z)), dz, 1e-5));
    // every row of (p - onehot) sums to zero: a softmax gradient taken on top of it would not leave it so
    orc_linear_backward(-1, 0, zs.data(), dz.data(), xs.data(), nullptr, w.data(), dw.data(), db.data(), batch, in_dim, classes);
    std::vector<float> w1 = w, b1 = bias;
    orc_sgd_update(0.1f, 0.0f, 0, 0.0f, dw.data(), (int64_t)w.size(), 1, w1.data(), nullptr);
    orc_sgd_update(0.1f, 0.0f, 0, 0.0f, db.data(), (int64_t)bias.size(), 1, b1.data(), nullptr);
    CHECK(close(to_host(instance.get_tensor_accessor(weights.at(0))), w1, 1e-5));
    CHECK(close(to_host(instance.get_tensor_accessor(weights.at(1))), b1, 1e-5));
    // an interior softmax (mean-squared error behind it) keeps the true gradient
    ComputationGraphBuilder b2;
    tensor_guid_t x2 = b2.create_input(shape({batch, classes}, DataType::FLOAT), CreateGrad::YES);
    tensor_guid_t p2 = b2.softmax(x2);
    auto target = random_vec(batch * classes, 43, 0.0f, 1.0f);
    auto TARGET = device_accessor(gpu, shape({batch, classes}, DataType::FLOAT), target);
    ComputationGraphInstance inst2 = create_computation_graph_instance(
        b2.computation_graph, optimizer, LossConfig{NonconfigurableLossAttrs{LossFunction::MEAN_SQUARED_ERROR_AVG_REDUCE}, TARGET, p2},
        {}, gpu, ProfilingSettings{0, 0}, handle, device_idx);
    GenericTensorAccessorW hx = cpu.allocate_tensor(inst2.get_tensor_accessor(x2).shape);
    memcpy(hx.ptr, zs.data(), zs.size() * 4);
    copy_accessor_data_to_l_from_r(inst2.get_tensor_accessor(x2), hx);
    perform_all_passes_for_computation_graph_instance(inst2, ProfilingSettings{0, 0}, handle, device_idx);
    std::vector<float> dp = to_host(*inst2.get_gradient_accessor(p2)), dx_want(zs.size());
    orc_softmax_backward(p.data(), dp.data(), dx_want.data(), batch, classes, 1);
    CHECK(close(to_host(*inst2.get_gradient_accessor(x2)), dx_want, 1e-5));
  });

  // Two Linear layers that share one bias tensor: both bias gradients are column reductions
  // whose last step the backward pass collects into one launch; they write the same tensor.
  run("Step driver: a bias shared by two Linear layers receives both gradients", [&] {
    int64_t batch = 64, dim = 96;
    ComputationGraph cg = make_empty_computation_graph();
    tensor_guid_t x = add_input_layer(cg, shape({batch, dim}, DataType::FLOAT)).outputs.at(0);
    tensor_guid_t w1 = add_weight_layer(cg, shape({dim, dim}, DataType::FLOAT)).outputs.at(0);
    tensor_guid_t w2 = add_weight_layer(cg, shape({dim, dim}, DataType::FLOAT)).outputs.at(0);
    tensor_guid_t bias = add_weight_layer(cg, shape({dim}, DataType::FLOAT)).outputs.at(0);
    LayerAttrs lin{LinearAttrs{(int)dim, true, DataType::FLOAT, std::nullopt, std::nullopt}, std::nullopt};
    tensor_guid_t h = add_layer(cg, lin, {x}, {w1, bias}).outputs.at(0);
    tensor_guid_t y = add_layer(cg, lin, {h}, {w2, bias}).outputs.at(0);
    auto xs = random_vec(batch * dim, 50), a1 = random_vec(dim * dim, 51, -0.2f, 0.2f), a2 = random_vec(dim * dim, 52, -0.2f, 0.2f),
         bs = random_vec(dim, 53), target = random_vec(batch * dim, 54);
    auto TARGET = device_accessor(gpu, shape({batch, dim}, DataType::FLOAT), target);
    device_id_t device_idx = make_device_id_t_from_idx(0, DeviceType::GPU);
    ComputationGraphInstance instance = create_computation_graph_instance(
        cg, OptimizerAttrs{SGDOptimizerAttrs{0.0, 0.0, false, 0.0}},
        LossConfig{NonconfigurableLossAttrs{LossFunction::MEAN_SQUARED_ERROR_AVG_REDUCE}, TARGET, y}, {}, gpu,
        ProfilingSettings{0, 0}, handle, device_idx);
    Allocator cpu = create_local_cpu_memory_allocator();
    auto put = [&](tensor_guid_t t, std::vector<float> const &v) {
      GenericTensorAccessorW hh = cpu.allocate_tensor(instance.get_tensor_accessor(t).shape);
      memcpy(hh.ptr, v.data(), v.size() * 4);
      copy_accessor_data_to_l_from_r(instance.get_tensor_accessor(t), hh);
    };
    put(x, xs); put(w1, a1); put(w2, a2); put(bias, bs);
    std::vector<float> hs(batch * dim), ys(batch * dim), dy(batch * dim), dh(batch * dim), dw(dim * dim), db2(dim), db1(dim);
    orc_linear_forward(-1, xs.data(), hs.data(), a1.data(), bs.data(), batch, dim, dim);
    orc_linear_forward(-1, hs.data(), ys.data(), a2.data(), bs.data(), batch, dim, dim);
    for (int step = 0; step < 2; step++) {  // the second step sees what the first left in the gradient
      perform_all_passes_for_computation_graph_instance(instance, ProfilingSettings{0, 0}, handle, device_idx);
      dy = to_host(*instance.get_gradient_accessor(y));
      orc_linear_backward(-1, 0, ys.data(), dy.data(), hs.data(), dh.data(), a2.data(), dw.data(), db2.data(), batch, dim, dim);
      orc_linear_backward(-1, 0, hs.data(), dh.data(), xs.data(), nullptr, a1.data(), dw.data(), db1.data(), batch, dim, dim);
      std::vector<float> want(dim);
      for (int64_t j = 0; j < dim; j++) want[j] = db1[j] + db2[j];
      CHECK(contains_non_zero(db1) && contains_non_zero(db2));
      CHECK(close(to_host(*instance.get_gradient_accessor(bias)), want, 1e-5));
    }
  });

  // The encoder layer of lib/models/src/models/transformer/transformer.cc:18-67 built through the
  // builder (BF16), a cast and a mean-squared-error loss behind it, Adam.  One step of the
  // instance must equal, bit for bit, the same operators called by hand with every gradient
  // added into zeroed memory: that pins the order, the placement, which gradients are
  // overwritten or cleared, the dropout streams and the mixed-precision update.
  run("Transformer encoder layer from the builder: one Adam step equals the hand-sequenced operators", [&] {
    int const B = 2, S = 24, E = 64, H = 4, FF = 256;  // head size FF / H = 64
    float const rate = 0.1f, eps = 1e-5f;
    ComputationGraphBuilder cgb;
    tensor_guid_t input = cgb.create_input(shape({B, S, E}, DataType::BF16), CreateGrad::NO);
    tensor_guid_t attn = cgb.multihead_attention(input, input, input, E, H, FF / H, FF / H, rate, false);
    CHECK(are_tensor_guid_shapes_equivalent(cgb.computation_graph, input, attn));
    tensor_guid_t res1 = cgb.add(attn, input);
    tensor_guid_t norm1 = cgb.layer_norm(res1, {-1}, true, eps);
    tensor_guid_t ff1 = cgb.dense(norm1, FF, Activation::RELU, true);
    tensor_guid_t drop1 = cgb.dropout(ff1, rate);
    tensor_guid_t ff2 = cgb.dense(drop1, E, std::nullopt, true);
    tensor_guid_t drop2 = cgb.dropout(ff2, rate);
    tensor_guid_t res2 = cgb.add(norm1, drop2);
    tensor_guid_t norm2 = cgb.layer_norm(res2, {-1}, true, eps);
    tensor_guid_t logits = cgb.cast(norm2, DataType::FLOAT);
    ComputationGraph const &cg = cgb.computation_graph;
    int64_t const n = (int64_t)B * S * E, nf = (int64_t)B * S * FF, M = B * S;

    auto LABEL = device_accessor(gpu, shape({B, S, E}, DataType::FLOAT), random_vec(n, 40));
    AdamOptimizerAttrs adam{1e-3, 0.9, 0.999, 1e-2, 1e-3, 0.9, 0.999, 1e-8};
    device_id_t device_idx = make_device_id_t_from_idx(0, DeviceType::GPU);
    ComputationGraphInstance inst = create_computation_graph_instance(
        cg, OptimizerAttrs{adam}, LossConfig{NonconfigurableLossAttrs{LossFunction::MEAN_SQUARED_ERROR_AVG_REDUCE}, LABEL, logits},
        {}, gpu, ProfilingSettings{0, 0}, handle, device_idx);

    // fill the input and every weight; keep device copies for the hand-sequenced run
    std::unordered_map<int, GenericTensorAccessorW> mine;  // tensor -> private copy
    unsigned seed = 50;
    auto init = [&](tensor_guid_t t, float lo, float hi) {
      TensorShape ts = inst.get_tensor_accessor(t).shape;
      GenericTensorAccessorW d = device_accessor(gpu, ts, random_vec((size_t)get_num_elements(ts.dims), seed++, lo, hi));
      copy_accessor_data_to_l_from_r(inst.get_tensor_accessor(t), d);
      mine[t.raw] = d;
    };
    init(input, -1.0f, 1.0f);
    std::vector<tensor_guid_t> weights;
    for (tensor_guid_t out : {attn, norm1, ff1, ff2, norm2}) {
      for (tensor_guid_t w : cgb.get_weights_of(out)) {
        weights.push_back(w);
        bool gamma = (out == norm1 || out == norm2) && w == cgb.get_weights_of(out)[0];
        init(w, gamma ? 0.5f : -0.2f, gamma ? 1.5f : 0.2f);
      }
    }
    CHECK(weights.size() == 9);

    perform_all_passes_for_computation_graph_instance(inst, ProfilingSettings{0, 0}, handle, device_idx);

    // ---- by hand ----
    ffk_stream_t st = stream.require_gpu();
    auto buf = [&](std::vector<int64_t> dims, DataType t) {
      GenericTensorAccessorW a = gpu.allocate_tensor(shape(dims, t));
      fill_with_zeros(a);
      return a;
    };
    auto W = [&](tensor_guid_t out, int i) { return mine.at(cgb.get_weights_of(out).at(i).raw); };
    std::unordered_map<int, GenericTensorAccessorW> dW;
    for (tensor_guid_t w : weights) dW[w.raw] = buf(mine.at(w.raw).shape.dims.ff_ordered, DataType::BF16);
    auto G = [&](tensor_guid_t out, int i) { return dW.at(cgb.get_weights_of(out).at(i).raw); };
    int const BT = FFK_BF16;
    auto x = mine.at(input.raw);
    auto a = buf({B, S, E}, DataType::BF16), r1 = buf({B, S, E}, DataType::BF16), n1 = buf({B, S, E}, DataType::BF16),
         f1 = buf({B, S, FF}, DataType::BF16), d1 = buf({B, S, FF}, DataType::BF16), f2 = buf({B, S, E}, DataType::BF16),
         d2 = buf({B, S, E}, DataType::BF16), r2 = buf({B, S, E}, DataType::BF16), n2 = buf({B, S, E}, DataType::BF16),
         lf = buf({B, S, E}, DataType::FLOAT);
    auto g_a = buf({B, S, E}, DataType::BF16), g_r1 = buf({B, S, E}, DataType::BF16), g_n1 = buf({B, S, E}, DataType::BF16),
         g_f1 = buf({B, S, FF}, DataType::BF16), g_d1 = buf({B, S, FF}, DataType::BF16), g_f2 = buf({B, S, E}, DataType::BF16),
         g_d2 = buf({B, S, E}, DataType::BF16), g_r2 = buf({B, S, E}, DataType::BF16), g_n2 = buf({B, S, E}, DataType::BF16),
         g_lf = buf({B, S, E}, DataType::FLOAT), g_x = buf({B, S, E}, DataType::BF16);
    ffk_mha_desc_t d{B, H, E, E, E, FF / H, FF / H, FF / H, E, S, S, 1.0f, 0};
    size_t reserve_bytes = ffk_mha_reserve_bytes(&d, BT);
    void *reserve = gpu.allocate(reserve_bytes);
    size_t ws_bytes = std::max({ffk_linear_backward_workspace_bytes(BT, FFK_ACT_RELU, 1, M, FF),
                                ffk_linear_backward_workspace_bytes(BT, FFK_ACT_NONE, 1, M, E),
                                ffk_layer_norm_backward_workspace_bytes(M, E)});
    void *ws = gpu.allocate(ws_bytes);
    auto stats = buf({4, M}, DataType::FLOAT);
    float *mean1 = stats.get_float_ptr(), *rstd1 = mean1 + M, *mean2 = mean1 + 2 * M, *rstd2 = mean1 + 3 * M;
    auto layer_of = [&](tensor_guid_t t) { return (uint64_t)cg.tensors.at(t.raw).source.raw; };
    auto ok = [&](int status) { check_ffk(status, "hand-sequenced step"); };
    ok(ffk_mha_forward(st, BT, &d, x.ptr, x.ptr, x.ptr, W(attn, 0).ptr, a.ptr, reserve, reserve_bytes));
    ok(ffk_element_binary_forward(st, BT, FFK_OP_EW_ADD, a.ptr, x.ptr, r1.ptr, n, n, n));
    ok(ffk_layer_norm_forward(st, BT, r1.ptr, n1.ptr, W(norm1, 0).ptr, W(norm1, 1).ptr, mean1, rstd1, M, E, eps));
    ok(ffk_linear_forward(st, BT, FFK_ACT_RELU, n1.ptr, f1.ptr, W(ff1, 0).ptr, W(ff1, 1).ptr, M, E, FF));
    ok(ffk_dropout_forward(st, BT, f1.ptr, d1.ptr, nf, rate, layer_of(drop1), 0));
    ok(ffk_linear_forward(st, BT, FFK_ACT_NONE, d1.ptr, f2.ptr, W(ff2, 0).ptr, W(ff2, 1).ptr, M, FF, E));
    ok(ffk_dropout_forward(st, BT, f2.ptr, d2.ptr, n, rate, layer_of(drop2), 0));
    ok(ffk_element_binary_forward(st, BT, FFK_OP_EW_ADD, n1.ptr, d2.ptr, r2.ptr, n, n, n));
    ok(ffk_layer_norm_forward(st, BT, r2.ptr, n2.ptr, W(norm2, 0).ptr, W(norm2, 1).ptr, mean2, rstd2, M, E, eps));
    ok(ffk_cast_forward(st, BT, FFK_FLOAT, n2.ptr, lf.ptr, n));
    ok(ffk_mean_squared_error_avg_loss_backward(st, g_lf.get_float_ptr(), lf.get_float_ptr(), LABEL.get_float_ptr(), n, n, 2.0f / n));
    ok(ffk_cast_backward(st, FFK_FLOAT, BT, g_lf.ptr, g_n2.ptr, n));
    ok(ffk_layer_norm_backward(st, BT, g_n2.ptr, r2.ptr, mean2, rstd2, W(norm2, 0).ptr, g_r2.ptr, G(norm2, 0).ptr, G(norm2, 1).ptr, M, E, ws, ws_bytes, 1));
    ok(ffk_element_binary_backward(st, BT, FFK_OP_EW_ADD, g_r2.ptr, n1.ptr, d2.ptr, g_n1.ptr, g_d2.ptr, n, 1));
    ok(ffk_dropout_backward(st, BT, g_d2.ptr, g_f2.ptr, n, rate, layer_of(drop2), 0, 1));
    ok(ffk_linear_backward(st, BT, FFK_ACT_NONE, 0, f2.ptr, g_f2.ptr, d1.ptr, g_d1.ptr, W(ff2, 0).ptr, G(ff2, 0).ptr, G(ff2, 1).ptr, M, FF, E, ws, ws_bytes, FFK_ACC_ALL));
    ok(ffk_dropout_backward(st, BT, g_d1.ptr, g_f1.ptr, nf, rate, layer_of(drop1), 0, 1));
    ok(ffk_linear_backward(st, BT, FFK_ACT_RELU, 0, f1.ptr, g_f1.ptr, n1.ptr, g_n1.ptr, W(ff1, 0).ptr, G(ff1, 0).ptr, G(ff1, 1).ptr, M, E, FF, ws, ws_bytes, FFK_ACC_ALL));
    ok(ffk_layer_norm_backward(st, BT, g_n1.ptr, r1.ptr, mean1, rstd1, W(norm1, 0).ptr, g_r1.ptr, G(norm1, 0).ptr, G(norm1, 1).ptr, M, E, ws, ws_bytes, 1));
    ok(ffk_element_binary_backward(st, BT, FFK_OP_EW_ADD, g_r1.ptr, a.ptr, x.ptr, g_a.ptr, g_x.ptr, n, 1));
    ok(ffk_mha_backward(st, BT, &d, x.ptr, g_x.ptr, x.ptr, nullptr, x.ptr, nullptr, W(attn, 0).ptr, G(attn, 0).ptr, g_a.ptr, reserve, reserve_bytes, 1));
    ok(ffk_stream_synchronize(st));

    CHECK(contains_non_zero(to_host(n2)));
    CHECK(to_host(inst.get_tensor_accessor(norm2)) == to_host(n2));
    CHECK(to_host(inst.get_tensor_accessor(drop1)) == to_host(d1));
    CHECK(to_host(*inst.get_gradient_accessor(norm1)) == to_host(g_n1));
    CHECK(to_host(*inst.get_gradient_accessor(attn)) == to_host(g_a));
    for (tensor_guid_t w : weights) {
      CHECK(contains_non_zero(to_host(dW.at(w.raw))));
      CHECK(to_host(*inst.get_gradient_accessor(w)) == to_host(dW.at(w.raw)));
    }
    // the update: fp32 master taken from the BF16 weights, Adam on it, BF16 copy rounded out
    for (tensor_guid_t w : weights) {
      int64_t nw = get_num_elements(mine.at(w.raw).shape.dims);
      auto master = buf({nw}, DataType::FLOAT), v = buf({nw}, DataType::FLOAT), m = buf({nw}, DataType::FLOAT);
      ok(ffk_cast_forward(st, BT, FFK_FLOAT, mine.at(w.raw).ptr, master.ptr, nw));
      ok(ffk_adam_update(st, BT, (float)adam.alpha_t, (float)adam.beta1, (float)adam.beta2, (float)adam.weight_decay,
                         (float)adam.epsilon, dW.at(w.raw).ptr, nw, 1, master.get_float_ptr(), v.get_float_ptr(),
                         m.get_float_ptr(), mine.at(w.raw).ptr));
      ok(ffk_stream_synchronize(st));
      CHECK(to_host(inst.get_tensor_accessor(w)) == to_host(mine.at(w.raw)));
      CHECK(to_host(*inst.get_master_weight_accessor(w)) == to_host(master));
    }
    // res1 = attn + input: attn's gradient has no other producer, so it is res1's gradient
    // memory itself; res2 = norm1 + drop2: drop2's likewise, norm1's (also fed by ff1) is added into
    CHECK(inst.get_gradient_accessor(attn)->ptr == inst.get_gradient_accessor(res1)->ptr);
    CHECK(inst.get_gradient_accessor(drop2)->ptr == inst.get_gradient_accessor(res2)->ptr);
    CHECK(inst.get_gradient_accessor(norm1)->ptr != inst.get_gradient_accessor(res2)->ptr);
    // all weights here are BF16 with stored gradients: one group, updated by one launch, so
    // value, gradient and master of every member lie at the same element offset of their arrays
    {
      tensor_guid_t w0 = weights.front();
      bool parallel = true;
      for (tensor_guid_t w : weights) {
        ptrdiff_t dv = (char *)inst.get_tensor_accessor(w).ptr - (char *)inst.get_tensor_accessor(w0).ptr;
        ptrdiff_t dg = (char *)inst.get_gradient_accessor(w)->ptr - (char *)inst.get_gradient_accessor(w0)->ptr;
        ptrdiff_t dm = (char *)inst.get_master_weight_accessor(w)->ptr - (char *)inst.get_master_weight_accessor(w0)->ptr;
        parallel = parallel && dv == dg && dm == 2 * dv && dv % 256 == 0;
      }
      CHECK(parallel);
    }
    // attrs advanced as lib/pcg/src/pcg/optimizer_attrs.cc:6-26 does
    AdamOptimizerAttrs next = std::get<AdamOptimizerAttrs>(inst.get_optimizer_attrs());
    CHECK(std::fabs(next.beta_t - 0.81) < 1e-12 && std::fabs(next.beta2_t - 0.999 * 0.999) < 1e-12);
    CHECK(std::fabs(next.alpha_t - 1e-3 * std::sqrt(1 - 0.999 * 0.999) / (1 - 0.81)) < 1e-15);
    // a second step draws different dropout masks (offset = iteration * elements)
    perform_forward_pass_for_computation_graph_instance(inst, ProfilingSettings{0, 0}, handle, device_idx);
    CHECK(!(to_host(inst.get_tensor_accessor(drop1)) == to_host(d1)));
  });
  // lib/kernels/test/src/test_concat_kernel.cc:8-117: four inputs, axis 0 and axis 1
  run("Concat forward/backward equal the oracle (the reference test's shapes)", [&] {
    for (int axis = 0; axis < 2; axis++) {
      int64_t rows = axis == 0 ? 2 : 4, cols = axis == 0 ? 4 : 2;
      TensorShape in_shape = shape({rows, cols}, DataType::FLOAT);
      TensorShape out_shape = axis == 0 ? shape({4 * rows, cols}, DataType::FLOAT) : shape({rows, 4 * cols}, DataType::FLOAT);
      std::vector<std::vector<float>> host;
      std::vector<GenericTensorAccessorR> ins;
      std::vector<GenericTensorAccessorW> grads;
      std::vector<float const *> hp;
      for (int i = 0; i < 4; i++) {
        host.push_back(random_vec(rows * cols, 60 + i));
        ins.push_back(device_accessor(gpu, in_shape, host.back()));
        grads.push_back(gpu.allocate_tensor(in_shape));
        fill_with_zeros(grads.back());
      }
      for (auto const &h : host) hp.push_back(h.data());
      int64_t blocks = axis == 0 ? 1 : rows, blk = axis == 0 ? rows * cols : cols;
      std::vector<int64_t> blks(4, blk);
      std::vector<float> want(4 * rows * cols);
      orc_concat_forward(want.data(), hp.data(), blks.data(), 4, blocks);
      auto OUT = gpu.allocate_tensor(out_shape);
      Kernels::Concat::forward_kernel(stream, OUT, ins, ff_dim_t{axis});
      CHECK(contains_non_zero(to_host(OUT)));
      CHECK(to_host(OUT) == want);
      Kernels::Concat::backward_kernel(stream, OUT, grads, ff_dim_t{axis});
      for (int i = 0; i < 4; i++) CHECK(to_host(grads[i]) == host[i]);  // split of the concatenation, added to zero
      CHECK_THROWS(Kernels::Concat::forward_kernel(stream, OUT, {ins[0], ins[1]}, ff_dim_t{axis}));
    }
  });

  // The graph of lib/models/src/models/dlrm/dlrm.cc:76-172 at a small size: embedding bags
  // (summed, BF16 out, cast to FLOAT), a bottom MLP on the dense features, the CAT
  // interaction, a top MLP; mean-squared-error loss, SGD.  One step against the oracle.
  run("DLRM-shaped graph (embedding bags, cast, concat, MLPs): one SGD step vs oracle", [&] {
    int64_t const B = 24, bag = 3, V = 50, D = 16, dense_in = 13, top = 32;
    int const tables = 3;
    ComputationGraphBuilder cgb;
    std::vector<tensor_guid_t> sparse, emb;
    for (int i = 0; i < tables; i++) {
      sparse.push_back(cgb.create_input(shape({B, bag}, DataType::INT64), CreateGrad::YES));
    }
    tensor_guid_t dense = cgb.create_input(shape({B, dense_in}, DataType::FLOAT), CreateGrad::YES);
    tensor_guid_t bottom = cgb.dense(dense, (int)D, Activation::RELU, true);
    for (int i = 0; i < tables; i++) {
      emb.push_back(cgb.cast(cgb.embedding(sparse[i], (int)V, (int)D, AggregateOp::SUM, DataType::BF16), DataType::FLOAT));
    }
    std::vector<tensor_guid_t> cat_in = {bottom};
    cat_in.insert(cat_in.end(), emb.begin(), emb.end());
    tensor_guid_t interact = cgb.concat(cat_in, 1);
    CHECK(cgb.get_shape(interact) == shape({B, D * (tables + 1)}, DataType::FLOAT));
    tensor_guid_t hidden = cgb.dense(interact, (int)top, Activation::RELU, true);
    tensor_guid_t out = cgb.dense(hidden, 1, Activation::RELU, true);

    auto label = random_vec(B, 70, 0.0f, 1.0f);
    auto LABEL = device_accessor(gpu, shape({B, 1}, DataType::FLOAT), label);
    device_id_t dev = make_device_id_t_from_idx(0, DeviceType::GPU);
    float const lr = 0.05f;
    ComputationGraphInstance inst = create_computation_graph_instance(
        cgb.computation_graph, OptimizerAttrs{SGDOptimizerAttrs{lr, 0.0, false, 0.0}},
        LossConfig{NonconfigurableLossAttrs{LossFunction::MEAN_SQUARED_ERROR_AVG_REDUCE}, LABEL, out}, {}, gpu,
        ProfilingSettings{0, 0}, handle, dev);

    Allocator cpu = create_local_cpu_memory_allocator();
    auto put = [&](tensor_guid_t t, std::vector<float> const &v) {
      GenericTensorAccessorW d = device_accessor(gpu, inst.get_tensor_accessor(t).shape, v);
      copy_accessor_data_to_l_from_r(inst.get_tensor_accessor(t), d);
    };
    std::vector<std::vector<int64_t>> idx(tables, std::vector<int64_t>(B * bag));
    std::mt19937 gen(7);
    for (int i = 0; i < tables; i++) {
      for (auto &v : idx[i]) v = gen() % V;
      GenericTensorAccessorW h = cpu.allocate_tensor(shape({B, bag}, DataType::INT64));
      memcpy(h.ptr, idx[i].data(), idx[i].size() * 8);
      copy_accessor_data_to_l_from_r(inst.get_tensor_accessor(sparse[i]), h);
    }
    auto x = random_vec(B * dense_in, 71);
    put(dense, x);
    auto wb = random_vec(D * dense_in, 72, -0.4f, 0.4f), bb = random_vec(D, 73, 0.0f, 0.2f);
    auto wh = random_vec(top * D * (tables + 1), 74, -0.2f, 0.2f), bh = random_vec(top, 75, 0.0f, 0.2f);
    auto wo = random_vec(top, 76, 0.0f, 0.3f), bo = random_vec(1, 77, 0.1f, 0.2f);
    put(cgb.get_weights_of(bottom)[0], wb); put(cgb.get_weights_of(bottom)[1], bb);
    put(cgb.get_weights_of(hidden)[0], wh); put(cgb.get_weights_of(hidden)[1], bh);
    put(cgb.get_weights_of(out)[0], wo); put(cgb.get_weights_of(out)[1], bo);
    std::vector<std::vector<float>> table(tables);
    std::vector<tensor_guid_t> table_guid;
    for (int i = 0; i < tables; i++) {
      table[i] = random_vec(V * D, 80 + i, -0.5f, 0.5f);
      table_guid.push_back(cgb.computation_graph.layers[cgb.computation_graph.tensors[emb[i].raw].source.raw].inputs[0]);
      table_guid[i] = cgb.get_weights_of(table_guid[i])[0];
      put(table_guid[i], table[i]);
    }

    perform_all_passes_for_computation_graph_instance(inst, ProfilingSettings{0, 0}, handle, dev);

    // oracle
    int64_t const W = D * (tables + 1);
    std::vector<float> bot(B * D), cat(B * W), hid(B * top), y(B), dy(B), dhid(B * top), dcat(B * W), dbot(B * D), dx(B * dense_in);
    std::vector<std::vector<float>> e(tables, std::vector<float>(B * D)), de(tables, std::vector<float>(B * D));
    orc_linear_forward(0, x.data(), bot.data(), wb.data(), bb.data(), B, dense_in, D);
    for (int i = 0; i < tables; i++) {
      orc_embedding_forward(idx[i].data(), e[i].data(), table[i].data(), 0, B, bag, D, V);
      orc_round_bf16_array(e[i].data(), e[i].size());
    }
    std::vector<float const *> parts = {bot.data()};
    for (auto const &v : e) parts.push_back(v.data());
    std::vector<int64_t> blks(tables + 1, D);
    orc_concat_forward(cat.data(), parts.data(), blks.data(), tables + 1, B);
    orc_linear_forward(0, cat.data(), hid.data(), wh.data(), bh.data(), B, W, top);
    orc_linear_forward(0, hid.data(), y.data(), wo.data(), bo.data(), B, top, 1);
    CHECK(close(to_host(inst.get_tensor_accessor(interact)), cat, 1e-5));
    CHECK(close(to_host(inst.get_tensor_accessor(out)), y, 1e-5) && contains_non_zero(y));
    orc_difference_loss_backward(dy.data(), y.data(), label.data(), B, 2.0f / B);
    std::vector<float> dwo(wo.size()), dbo(1), dwh(wh.size()), dbh(top), dwb(wb.size()), dbb(D);
    orc_linear_backward(0, 0, y.data(), dy.data(), hid.data(), dhid.data(), wo.data(), dwo.data(), dbo.data(), B, top, 1);
    orc_linear_backward(0, 0, hid.data(), dhid.data(), cat.data(), dcat.data(), wh.data(), dwh.data(), dbh.data(), B, W, top);
    std::vector<float *> dparts = {dbot.data()};
    for (auto &v : de) dparts.push_back(v.data());
    orc_concat_backward(dcat.data(), dparts.data(), blks.data(), tables + 1, B, 0);
    orc_linear_backward(0, 0, bot.data(), dbot.data(), x.data(), dx.data(), wb.data(), dwb.data(), dbb.data(), B, dense_in, D);
    CHECK(close(to_host(*inst.get_gradient_accessor(cgb.get_weights_of(hidden)[0])), dwh, 1e-5));
    CHECK(close(to_host(*inst.get_gradient_accessor(cgb.get_weights_of(bottom)[0])), dwb, 1e-5));
    CHECK(close(to_host(*inst.get_gradient_accessor(cgb.get_weights_of(bottom)[1])), dbb, 1e-5));
    CHECK(close(to_host(*inst.get_gradient_accessor(dense)), dx, 1e-5));
    for (int i = 0; i < tables; i++) {
      // the cast's backward rounds the gradient to BF16 before the scatter-add, so an fp32
      // last-bit difference upstream can move an addend by one BF16 step: BF16 tolerance
      orc_round_bf16_array(de[i].data(), de[i].size());
      std::vector<float> dtab(V * D, 0.0f);
      orc_embedding_backward_f64(idx[i].data(), de[i].data(), dtab.data(), 0, B, bag, D, V);
      CHECK(contains_non_zero(dtab));
      CHECK(close(to_host(*inst.get_gradient_accessor(table_guid[i])), dtab, 2e-2));
      for (size_t j = 0; j < dtab.size(); j++) table[i][j] -= lr * dtab[j];
      CHECK(close(to_host(inst.get_tensor_accessor(table_guid[i])), table[i], 1e-4));
    }
    for (size_t j = 0; j < wh.size(); j++) wh[j] -= lr * dwh[j];
    CHECK(close(to_host(inst.get_tensor_accessor(cgb.get_weights_of(hidden)[0])), wh, 1e-5));
  });
  run("Transpose, Reshape, Split and Gather equal the oracle", [&] {
    // transpose [4, 6, 10] -> perm (2, 0, 1), and its backward into a non-zero gradient
    std::vector<int64_t> dims = {4, 6, 10};
    TransposeAttrs tattrs{{2, 0, 1}};
    int64_t const n = 4 * 6 * 10;
    auto x = random_vec(n, 90), old = random_vec(n, 91), dout = random_vec(n, 92);
    auto X = device_accessor(gpu, shape(dims, DataType::FLOAT), x);
    auto Y = gpu.allocate_tensor(shape({10, 4, 6}, DataType::FLOAT));
    Kernels::Transpose::forward_kernel(stream, tattrs, X, Y);
    std::vector<float> want(n);
    orc_transpose_nd(x.data(), want.data(), 3, dims.data(), tattrs.permutation.data(), 0);
    CHECK(to_host(Y) == want);
    auto DY = device_accessor(gpu, Y.shape, dout);
    auto DX = device_accessor(gpu, X.shape, old);
    Kernels::Transpose::backward_kernel(stream, tattrs, DY, DX);
    std::vector<int64_t> odims = {10, 4, 6};
    int inverse[3] = {1, 2, 0};
    std::vector<float> wantb = old;
    orc_transpose_nd(dout.data(), wantb.data(), 3, odims.data(), inverse, 1);
    CHECK(to_host(DX) == wantb);
    CHECK_THROWS(Kernels::Transpose::forward_kernel(stream, TransposeAttrs{{0, 1, 2}}, X, Y));  // dims do not match

    // reshape: same elements
    auto R = gpu.allocate_tensor(shape({24, 10}, DataType::FLOAT));
    Kernels::Reshape::forward_kernel(stream, X, R);
    CHECK(to_host(R) == x);
    Kernels::Reshape::backward_kernel(stream, R, DX);
    for (int64_t i = 0; i < n; i++) wantb[i] += x[i];
    CHECK(to_host(DX) == wantb);

    // split [6, 10] into column blocks 3 | 7, then back
    auto IN = device_accessor(gpu, shape({6, 10}, DataType::FLOAT), random_vec(60, 93));
    auto O1 = gpu.allocate_tensor(shape({6, 3}, DataType::FLOAT)), O2 = gpu.allocate_tensor(shape({6, 7}, DataType::FLOAT));
    float *outs[2] = {O1.get_float_ptr(), O2.get_float_ptr()};
    int blk[2] = {3, 7};
    Kernels::Split::forward_kernel(stream, outs, IN.get_float_ptr(), blk, 10, 6, 2);
    auto in_host = to_host(IN), o1 = to_host(O1), o2 = to_host(O2);
    bool split_ok = true;
    for (int r = 0; r < 6; r++) {
      for (int c = 0; c < 10; c++) split_ok = split_ok && in_host[r * 10 + c] == (c < 3 ? o1[r * 3 + c] : o2[r * 7 + c - 3]);
    }
    CHECK(split_ok);
    auto DIN = gpu.allocate_tensor(IN.shape);
    fill_with_zeros(DIN);
    float const *grads[2] = {O1.get_float_ptr(), O2.get_float_ptr()};
    Kernels::Split::backward_kernel(stream, DIN.get_float_ptr(), grads, blk, 10, 6, 2);
    CHECK(to_host(DIN) == in_host);

    // gather along dim 1 of [4, 6, 10] with an int32 index [4, 3, 10]
    std::vector<int64_t> idx(4 * 3 * 10);
    std::mt19937 gen(3);
    for (auto &v : idx) v = gen() % 6;
    std::vector<int32_t> idx32(idx.begin(), idx.end());
    Allocator cpu = create_local_cpu_memory_allocator();
    GenericTensorAccessorW hidx = cpu.allocate_tensor(shape({4, 3, 10}, DataType::INT32));
    memcpy(hidx.ptr, idx32.data(), idx32.size() * 4);
    GenericTensorAccessorW I = copy_tensor_accessor_w(hidx, gpu);
    auto gstate = Kernels::Gather::init_kernel(DeviceType::GPU, handle, ff_dim_t{1});
    auto G = gpu.allocate_tensor(shape({4, 3, 10}, DataType::FLOAT));
    Kernels::Gather::forward_kernel(stream, gstate, X, I, G);
    std::vector<float> gwant(idx.size());
    orc_gather_forward(x.data(), idx.data(), gwant.data(), 4, 6, 3, 10);
    CHECK(to_host(G) == gwant && contains_non_zero(gwant));
    auto gd = random_vec(idx.size(), 94);
    auto GD = device_accessor(gpu, G.shape, gd);
    auto DXg = device_accessor(gpu, X.shape, old);
    Kernels::Gather::backward_kernel(stream, gstate, GD, I, DXg);
    std::vector<float> gb = old;
    orc_gather_backward(gd.data(), idx.data(), gb.data(), 4, 6, 3, 10);
    CHECK(close(to_host(DXg), gb, 1e-5));
  });

  run("Step driver: transpose, reshape and gather layers carry values and gradients", [&] {
    // y = gather(reshape(transpose(x, (1, 0, 2)), [6, 40]), index, dim 1); loss gradient = 1 / batch
    ComputationGraphBuilder cgb;
    tensor_guid_t x = cgb.create_input(shape({4, 6, 10}, DataType::FLOAT), CreateGrad::YES);
    tensor_guid_t index = cgb.create_input(shape({6, 5}, DataType::INT64), CreateGrad::NO);
    tensor_guid_t t = cgb.transpose(x, {1, 0, 2});
    tensor_guid_t r = cgb.reshape(t, {6, 40});
    tensor_guid_t y = cgb.gather(r, index, 1);
    CHECK(cgb.get_shape(y) == shape({6, 5}, DataType::FLOAT));
    device_id_t dev = make_device_id_t_from_idx(0, DeviceType::GPU);
    auto LABEL = gpu.allocate_tensor(shape({6, 5}, DataType::FLOAT));
    ComputationGraphInstance inst = create_computation_graph_instance(
        cgb.computation_graph, OptimizerAttrs{SGDOptimizerAttrs{0.1, 0.0, false, 0.0}},
        LossConfig{NonconfigurableLossAttrs{LossFunction::IDENTITY}, LABEL, y}, {}, gpu, ProfilingSettings{0, 0}, handle, dev);
    auto xv = random_vec(240, 95);
    copy_accessor_data_to_l_from_r(inst.get_tensor_accessor(x), device_accessor(gpu, shape({4, 6, 10}, DataType::FLOAT), xv));
    std::vector<int64_t> idx(30);
    std::mt19937 gen(5);
    for (auto &v : idx) v = gen() % 40;
    Allocator cpu = create_local_cpu_memory_allocator();
    GenericTensorAccessorW hidx = cpu.allocate_tensor(shape({6, 5}, DataType::INT64));
    memcpy(hidx.ptr, idx.data(), idx.size() * 8);
    copy_accessor_data_to_l_from_r(inst.get_tensor_accessor(index), hidx);
    perform_all_passes_for_computation_graph_instance(inst, ProfilingSettings{0, 0}, handle, dev);
    // oracle: the same three steps, and the scatter / reshape / inverse transpose of a constant gradient
    std::vector<int64_t> dims = {4, 6, 10}, tdims = {6, 4, 10};
    int perm[3] = {1, 0, 2};
    std::vector<float> tv(240), yv(30), dy(30, 1.0f / 6.0f), dr(240, 0.0f), dxw(240);
    orc_transpose_nd(xv.data(), tv.data(), 3, dims.data(), perm, 0);
    orc_gather_forward(tv.data(), idx.data(), yv.data(), 6, 40, 5, 1);
    CHECK(to_host(inst.get_tensor_accessor(y)) == yv);
    orc_gather_backward(dy.data(), idx.data(), dr.data(), 6, 40, 5, 1);
    orc_transpose_nd(dr.data(), dxw.data(), 3, tdims.data(), perm, 0);  // (1, 0, 2) is its own inverse
    CHECK(close(to_host(*inst.get_gradient_accessor(x)), dxw, 1e-6) && contains_non_zero(dxw));
  });
  run("Step driver: fused operator pairs give the bits of one kernel per operator", [&] {
    // x -> dense -> GELU -> dropout -> dense -> dropout -> (+ x) -> cast -> loss; two instances of the
    // same graph, one created with FFK_OPTION_LAYER_UNFUSED set, stepped twice each (the second step uses
    // the next dropout offsets)
    // ... at a size whose Linears run the two element-wise launches themselves, and at one where
    // the library applies the pairs on the GEMMs' tile stores
    for (int big = 0; big < 2; big++) {
    int64_t const B = big ? 2048 : 16, E = big ? 1024 : 64, FF = big ? 2048 : 128;
    float const init = big ? 0.05f : 0.3f;
    auto build = [&](ComputationGraphBuilder &cgb, tensor_guid_t &x, tensor_guid_t &logits, std::vector<tensor_guid_t> &ws) {
      x = cgb.create_input(shape({B, E}, DataType::BF16), CreateGrad::YES);
      tensor_guid_t h = cgb.dense(x, (int)FF, Activation::GELU, true);
      ws = {};  // collected below: every weight tensor of the graph
      tensor_guid_t d1 = cgb.dropout(h, 0.25f);
      tensor_guid_t f2 = cgb.dense(d1, (int)E, std::nullopt, true);
      tensor_guid_t r = cgb.add(cgb.dropout(f2, 0.25f), x);
      logits = cgb.cast(r, DataType::FLOAT);
    };
    device_id_t dev = make_device_id_t_from_idx(0, DeviceType::GPU);
    auto LABEL = device_accessor(gpu, shape({B, E}, DataType::FLOAT), random_vec(B * E, 71));
    std::vector<std::vector<float>> results[2];
    auto ok = [](int rc) {
      if (rc != FFK_OK) throw std::runtime_error(ffk_last_error());
    };
    for (int unfused = 0; unfused < 2; unfused++) {
      ComputationGraphBuilder cgb;
      tensor_guid_t x, logits;
      std::vector<tensor_guid_t> ws;
      build(cgb, x, logits, ws);
      if (unfused) ffk_set_option(FFK_OPTION_LAYER_UNFUSED, 1);
      ComputationGraphInstance inst = create_computation_graph_instance(
          cgb.computation_graph, OptimizerAttrs{SGDOptimizerAttrs{0.05, 0.9, false, 0.0}},
          LossConfig{NonconfigurableLossAttrs{LossFunction::MEAN_SQUARED_ERROR_AVG_REDUCE}, LABEL, logits}, {}, gpu,
          ProfilingSettings{0, 0}, handle, dev);
      if (unfused) ffk_set_option(FFK_OPTION_LAYER_UNFUSED, 0);
      // the GELU of dense(.., GELU) is its own layer: find the weights by layer order (same in both graphs)
      int seed = 80;
      for (size_t t = 0; t < cgb.computation_graph.tensors.size(); t++) {
        tensor_guid_t g{(int)t};
        auto const &src = cgb.computation_graph.layers.at(cgb.computation_graph.tensors[t].source.raw);
        bool const weight = std::holds_alternative<WeightAttrs>(src.attrs.op_attrs);
        if (!weight && !(g == x)) continue;
        if (weight) ws.push_back(g);
        TensorShape s16 = cgb.computation_graph.tensors[t].shape;
        auto host = random_vec(get_num_elements(s16.dims), seed++);
        for (auto &v : host) v *= init;
        auto f32 = device_accessor(gpu, TensorShape{s16.dims, DataType::FLOAT}, host);
        ok(ffk_cast_forward(nullptr, FFK_FLOAT, FFK_BF16, f32.ptr, inst.get_tensor_accessor(g).ptr, get_num_elements(s16.dims)));
      }
      ok(ffk_stream_synchronize(nullptr));
      for (int step = 0; step < 2; step++) perform_all_passes_for_computation_graph_instance(inst, ProfilingSettings{0, 0}, handle, dev);
      results[unfused].push_back(to_host(inst.get_tensor_accessor(logits)));
      results[unfused].push_back(to_host(*inst.get_gradient_accessor(x)));
      for (tensor_guid_t w : ws) results[unfused].push_back(to_host(inst.get_tensor_accessor(w)));
    }
    CHECK(results[0].size() == results[1].size() && results[0].size() == 6);
    for (size_t i = 0; i < results[0].size(); i++) {
      CHECK(contains_non_zero(results[0][i]));
      CHECK(results[0][i] == results[1][i]);
    }
    }
  });

  // The encoder layer of the reference's transformer builder with its default configuration
  // (lib/models/src/models/transformer/transformer.cc:6-16,32-67): 512 features, 8 heads,
  // kdim = vdim = dim_feedforward / num_heads = 256, feed-forward 2048 with ReLU, dropout 0.1,
  // LayerNorm after each residual add.  FLOAT (the reference's data type) and BF16.
  run("The reference's default transformer encoder layer (512 features, 8 heads x 256, FFN 2048): steps, fused = unfused, loss falls", [&] {
    int64_t const B = 2, S = 40, E = 512, FF = 2048;
    int const H = 8, KD = (int)(FF / H);
    float const rate = 0.1f, eps = 1e-5f;
    for (DataType type : {DataType::FLOAT, DataType::BF16}) {
      tensor_guid_t x, out;
      auto build = [&](ComputationGraphBuilder &cgb) {
        x = cgb.create_input(shape({B, S, E}, type), CreateGrad::YES);
        tensor_guid_t attn = cgb.multihead_attention(x, x, x, (int)E, H, KD, KD, rate, false);
        tensor_guid_t n1 = cgb.layer_norm(cgb.add(attn, x), {-1}, true, eps);
        tensor_guid_t ff1 = cgb.dropout(cgb.dense(n1, (int)FF, Activation::RELU, true), rate);
        tensor_guid_t ff2 = cgb.dropout(cgb.dense(ff1, (int)E, std::nullopt, true), rate);
        tensor_guid_t n2 = cgb.layer_norm(cgb.add(n1, ff2), {-1}, true, eps);
        out = type == DataType::FLOAT ? n2 : cgb.cast(n2, DataType::FLOAT);
      };
      device_id_t dev = make_device_id_t_from_idx(0, DeviceType::GPU);
      auto label = random_vec(B * S * E, 401);
      auto LABEL = device_accessor(gpu, shape({B, S, E}, DataType::FLOAT), label);
      auto loss_of = [&](std::vector<float> const &o) {
        double l = 0;
        for (size_t i = 0; i < o.size(); i++) l += ((double)o[i] - label[i]) * ((double)o[i] - label[i]);
        return l / (double)o.size();
      };
      std::vector<std::vector<float>> results[2];
      std::vector<double> losses;
      for (int unfused = 0; unfused < 2; unfused++) {
        ComputationGraphBuilder cgb;
        build(cgb);
        // the attention layer's weight has the reference's element count (attention.cc:165-185)
        if (unfused) ffk_set_option(FFK_OPTION_LAYER_UNFUSED, 1);
        ComputationGraphInstance inst = create_computation_graph_instance(
            cgb.computation_graph, OptimizerAttrs{SGDOptimizerAttrs{0.05, 0.9, false, 0.0}},
            LossConfig{NonconfigurableLossAttrs{LossFunction::MEAN_SQUARED_ERROR_AVG_REDUCE}, LABEL, out}, {}, gpu,
            ProfilingSettings{0, 0}, handle, dev);
        if (unfused) ffk_set_option(FFK_OPTION_LAYER_UNFUSED, 0);
        std::vector<tensor_guid_t> ws;
        unsigned seed = 500;
        for (size_t t = 0; t < cgb.computation_graph.tensors.size(); t++) {
          tensor_guid_t g{(int)t};
          auto const &src = cgb.computation_graph.layers.at(cgb.computation_graph.tensors[t].source.raw);
          bool const weight = std::holds_alternative<WeightAttrs>(src.attrs.op_attrs);
          if (!weight && !(g == x)) continue;
          if (weight) ws.push_back(g);
          TensorShape ts = cgb.computation_graph.tensors[t].shape;
          bool const vec = weight && ts.dims.ff_ordered.size() == 1 && get_num_elements(ts.dims) <= FF;
          auto host = g == x ? random_vec((size_t)get_num_elements(ts.dims), seed++)
                             : random_vec((size_t)get_num_elements(ts.dims), seed++, vec ? 0.5f : -0.05f, vec ? 1.5f : 0.05f);
          copy_accessor_data_to_l_from_r(inst.get_tensor_accessor(g), device_accessor(gpu, ts, host));
        }
        if (!unfused) {
          // 3 * (512 * 256) * 8 + 512 * 256 * 8 elements
          size_t attn_w = 0;
          for (tensor_guid_t w : ws) attn_w = std::max(attn_w, (size_t)get_num_elements(cgb.computation_graph.tensors[w.raw].shape.dims));
          CHECK(attn_w == (size_t)(4 * E * KD * H));
        }
        for (int step = 0; step < (unfused ? 3 : 6); step++) {
          perform_all_passes_for_computation_graph_instance(inst, ProfilingSettings{0, 0}, handle, dev);
          if (step == 2) {
            results[unfused].push_back(to_host(inst.get_tensor_accessor(out)));
            results[unfused].push_back(to_host(*inst.get_gradient_accessor(x)));
            for (tensor_guid_t w : ws) results[unfused].push_back(to_host(inst.get_tensor_accessor(w)));
          }
          if (!unfused) losses.push_back(loss_of(to_host(inst.get_tensor_accessor(out))));
        }
      }
      CHECK(results[0].size() == results[1].size() && results[0].size() == 11);
      for (size_t i = 0; i < results[0].size(); i++) {
        CHECK(contains_non_zero(results[0][i]));
        bool finite = true;
        for (float v : results[0][i]) finite = finite && std::isfinite(v);
        CHECK(finite);
        CHECK(results[0][i] == results[1][i]);
      }
      CHECK(losses.size() == 6 && std::isfinite(losses[5]));
      CHECK(losses[5] < losses[0]);
      printf("    %s loss per step: %.4f %.4f %.4f %.4f %.4f %.4f\n", type == DataType::FLOAT ? "fp32" : "bf16", losses[0],
             losses[1], losses[2], losses[3], losses[4], losses[5]);
    }
  });

  // Token embedding -> encoder layer -> vocabulary projection -> softmax -> sparse cross entropy:
  // the shape of the reference's BERT builder (lib/models/src/models/bert/bert.cc) at toy size.
  // Two instances, one created with one kernel per operator: the planner's fusions must not change
  // a bit over three steps, and three more steps on the same batch must bring the loss down.
  run("BERT-shaped graph (embedding, attention, FFN, vocabulary softmax, sparse CE): fused = unfused, loss falls", [&] {
    int64_t const B = 2, S = 24, E = 64, FF = 256, V = 96, T = B * S;
    int const H = 2, HD = 64;
    float const rate = 0.1f, eps = 1e-5f;
    tensor_guid_t ids, prob;
    auto build = [&](ComputationGraphBuilder &cgb) {
      ids = cgb.create_input(shape({B, S}, DataType::INT32), CreateGrad::NO);
      tensor_guid_t tok = cgb.embedding(ids, (int)V, (int)E, std::nullopt, DataType::BF16);
      tensor_guid_t attn = cgb.multihead_attention(tok, tok, tok, (int)E, H, HD, HD, rate, false);
      tensor_guid_t n1 = cgb.layer_norm(cgb.add(attn, tok), {-1}, true, eps);
      tensor_guid_t ff1 = cgb.dropout(cgb.dense(n1, (int)FF, Activation::GELU, true), rate);
      tensor_guid_t ff2 = cgb.dropout(cgb.dense(ff1, (int)E, std::nullopt, true), rate);
      tensor_guid_t n2 = cgb.layer_norm(cgb.add(n1, ff2), {-1}, true, eps);
      tensor_guid_t logits = cgb.dense(cgb.reshape(n2, {T, E}), (int)V, std::nullopt, true);
      prob = cgb.softmax(cgb.cast(logits, DataType::FLOAT));
    };
    std::vector<int> id_host(T), label_host(T);
    for (int64_t i = 0; i < T; i++) {
      id_host[i] = (int)((i * 37 + 11) % V);
      label_host[i] = (int)((i * 53 + 7) % V);
    }
    Allocator cpu = create_local_cpu_memory_allocator();
    GenericTensorAccessorW hl = cpu.allocate_tensor(shape({T}, DataType::INT32));
    memcpy(hl.ptr, label_host.data(), label_host.size() * 4);
    GenericTensorAccessorW LABEL = copy_tensor_accessor_w(hl, gpu);
    device_id_t dev = make_device_id_t_from_idx(0, DeviceType::GPU);
    auto loss_of = [&](std::vector<float> const &p) {
      double l = 0;
      for (int64_t i = 0; i < T; i++) l -= std::log((double)p[i * V + label_host[i]] + 1e-30);
      return l / T;
    };
    std::vector<std::vector<float>> results[2];
    std::vector<double> losses;
    for (int unfused = 0; unfused < 2; unfused++) {
      ComputationGraphBuilder cgb;
      build(cgb);
      if (unfused) ffk_set_option(FFK_OPTION_LAYER_UNFUSED, 1);
      ComputationGraphInstance inst = create_computation_graph_instance(
          cgb.computation_graph, OptimizerAttrs{SGDOptimizerAttrs{0.1, 0.9, false, 0.0}},
          LossConfig{SparseCategoricalCrossEntropyLossAttrs{false}, LABEL, prob}, {}, gpu, ProfilingSettings{0, 0}, handle, dev);
      if (unfused) ffk_set_option(FFK_OPTION_LAYER_UNFUSED, 0);
      GenericTensorAccessorW hi = cpu.allocate_tensor(shape({B, S}, DataType::INT32));
      memcpy(hi.ptr, id_host.data(), id_host.size() * 4);
      copy_accessor_data_to_l_from_r(inst.get_tensor_accessor(ids), hi);
      std::vector<tensor_guid_t> ws;
      unsigned seed = 300;
      for (size_t t = 0; t < cgb.computation_graph.tensors.size(); t++) {
        tensor_guid_t g{(int)t};
        auto const &src = cgb.computation_graph.layers.at(cgb.computation_graph.tensors[t].source.raw);
        if (!std::holds_alternative<WeightAttrs>(src.attrs.op_attrs)) continue;
        ws.push_back(g);
        TensorShape ts = cgb.computation_graph.tensors[t].shape;
        // one-dimensional weights are biases and LayerNorm parameters: around 1 keeps the scales alive
        bool const vec = ts.dims.ff_ordered.size() == 1;
        auto host = random_vec((size_t)get_num_elements(ts.dims), seed++, vec ? 0.5f : -0.2f, vec ? 1.5f : 0.2f);
        copy_accessor_data_to_l_from_r(inst.get_tensor_accessor(g), device_accessor(gpu, ts, host));
      }
      for (int step = 0; step < (unfused ? 3 : 6); step++) {
        perform_all_passes_for_computation_graph_instance(inst, ProfilingSettings{0, 0}, handle, dev);
        if (step == 2) {
          results[unfused].push_back(to_host(inst.get_tensor_accessor(prob)));
          for (tensor_guid_t w : ws) results[unfused].push_back(to_host(inst.get_tensor_accessor(w)));
        }
        if (!unfused) losses.push_back(loss_of(to_host(inst.get_tensor_accessor(prob))));
      }
    }
    CHECK(results[0].size() == results[1].size() && results[0].size() > 10);
    for (size_t i = 0; i < results[0].size(); i++) {
      CHECK(contains_non_zero(results[0][i]));
      CHECK(results[0][i] == results[1][i]);
    }
    CHECK(losses.size() == 6 && std::isfinite(losses[5]));
    CHECK(losses[5] < losses[0]);
    printf("    loss per step: %.4f %.4f %.4f %.4f %.4f %.4f\n", losses[0], losses[1], losses[2], losses[3], losses[4], losses[5]);
  });
}

int main(int argc, char **argv) {
  std::string mode = argc > 1 ? argv[1] : "--cpu";
  if (mode == "--cpu") {
    cpu_tests();
  } else if (mode == "--gpu") {
    gpu_tests();
  } else {
    printf("usage: test_host --cpu | --gpu\n");
    return 2;
  }
  printf("%d checks, %d failed\n", g_checks, g_failed);
  return g_failed == 0 ? 0 : 1;
}
