// A translation unit written the way a caller inside the reference is: only the
// include lines the reference's own files use for this path
// (lib/task-spec/src/task-spec/ops/impl/{element_unary,element_binary,gather,
// transpose,linear}.cc:1-20, lib/local-execution and lib/kernels/test/src) and
// the accessor calls of lib/kernels/include/kernels/accessor.h:24-57
// (get<DataType>(), at<DataType>()).  Compiling it is half of the check; the
// function below runs a Linear known-answer case, an ElementUnary, a Transpose
// and a Gather through those names and reports what disagrees.
#include "kernels/accessor.h"
#include "kernels/allocation.h"
#include "kernels/copy_tensor_accessor.h"
#include "kernels/create_local_allocator_for_device_type.h"
#include "kernels/device.h"
#include "kernels/device_handle_t.dtg.h"
#include "kernels/device_stream_t.dtg.h"
#include "kernels/element_binary_kernels.h"
#include "kernels/element_unary_kernels.h"
#include "kernels/ff_handle.h"
#include "kernels/gather_kernels.h"
#include "kernels/linear_kernels.h"
#include "kernels/local_cpu_allocator.h"
#include "kernels/local_cuda_allocator.h"
#include "kernels/managed_ff_stream.h"
#include "kernels/managed_per_device_ff_handle.h"
#include "kernels/profiling.h"
#include "kernels/profiling_settings.dtg.h"
#include "kernels/reshape_kernels.h"
#include "kernels/split_kernels.h"
#include "kernels/transpose_kernels.h"
#include "op-attrs/datatype.dtg.h"
#include "op-attrs/tensor_shape.dtg.h"
#include "pcg/device_type.dtg.h"
#include <string>

using namespace FlexFlow;

static GenericTensorAccessorW on_device(Allocator &gpu, Allocator &cpu, TensorShape const &shape, std::vector<float> const &v) {
  GenericTensorAccessorW h = cpu.allocate_tensor(shape);
  float *p = h.get<DataType::FLOAT>();
  for (size_t i = 0; i < v.size(); i++) p[i] = v[i];
  return copy_tensor_accessor_w(h, gpu);
}

// Returns the empty string when every check holds, else what failed.
std::string reference_style_translation_unit() {
  std::string bad;
  auto expect = [&](bool ok, char const *what) {
    if (!ok) bad += std::string(bad.empty() ? "" : "; ") + what;
  };
  ManagedFFStream managed_stream{};
  ManagedPerDeviceFFHandle managed_handle = initialize_single_gpu_handle(1024 * 1024, true);
  device_handle_t handle = device_handle_t_from_managed_ff_handle(managed_handle);
  device_stream_t stream = get_gpu_device_stream();
  Allocator gpu = create_local_allocator_for_device_type(DeviceType::GPU);
  Allocator cpu = create_local_cpu_memory_allocator();

  // Linear, the reference's known-answer case (lib/kernels/test/src/kernels/linear_kernels_cpu.cc:11-66)
  TensorShape xs{TensorDims{{4, 3}}, DataType::FLOAT}, ws{TensorDims{{2, 3}}, DataType::FLOAT};
  TensorShape bs{TensorDims{{2}}, DataType::FLOAT}, ys{TensorDims{{4, 2}}, DataType::FLOAT};
  GenericTensorAccessorW X = on_device(gpu, cpu, xs, {3, 3, 6, 2, 1, 5, 1, 2, -2, 8, 0.5, -3});
  GenericTensorAccessorW W = on_device(gpu, cpu, ws, {1, 2, 1.5, 0.5, 4, -1});
  GenericTensorAccessorW B = on_device(gpu, cpu, bs, {3, -1});
  GenericTensorAccessorW Y = gpu.allocate_tensor(ys);
  LinearAttrs attrs{2, true, DataType::FLOAT, std::nullopt, std::nullopt};
  std::optional<LinearPerDeviceState> state = linear_init_kernel(
      DeviceType::GPU, handle, std::nullopt, std::nullopt, true, DataType::FLOAT, DataType::FLOAT, DataType::FLOAT, 4, 2);
  linear_forward_kernel(stream, state, attrs, X, Y, W, GenericTensorAccessorR(B));
  GenericTensorAccessorR Yh = copy_tensor_accessor_r_to_cpu_if_necessary(Y, cpu);
  float const want[4][2] = {{21, 6.5}, {14.5, -1}, {5, 9.5}, {7.5, 8}};
  for (int64_t i = 0; i < 4; i++) {
    for (int64_t j = 0; j < 2; j++) expect(Yh.at<DataType::FLOAT>({i, j}) == want[i][j], "Linear known answer through at<DataType::FLOAT>");
  }
  expect(Yh.get<DataType::FLOAT>() == Yh.get_float_ptr(), "get<DataType::FLOAT> is the float pointer");
  bool threw = false;
  try {
    (void)Yh.get<DataType::INT32>();
  } catch (std::exception const &) {
    threw = true;
  }
  expect(threw, "get<DataType::INT32> on a FLOAT accessor is refused");
  threw = false;
  try {
    (void)GenericTensorAccessorR(Y).at<DataType::FLOAT>({0, 0});  // device-resident
  } catch (std::exception const &) {
    threw = true;
  }
  expect(threw, "at<> on a device accessor is refused");
  expect(copy_tensor_accessor_r_to_cpu_if_necessary(Yh, cpu).ptr == Yh.ptr, "a host accessor is returned as it is");
  linear_cleanup_kernel(DeviceType::GPU, state);

  // ElementUnary: scalar multiply by 2 (element_unary.cc:36-52 of the task implementation)
  {
    using namespace FlexFlow::Kernels::ElementUnary;
    ElementUnaryAttrs ua{OperatorType::SCALAR_MULTIPLY, 2.0f};
    std::optional<ElementUnaryPerDeviceState> us = init_kernel(DeviceType::GPU, ys, ys, ua);
    GenericTensorAccessorW Z = gpu.allocate_tensor(ys);
    forward_kernel(stream, us, ua, handle, Y, Z);
    GenericTensorAccessorW Zh = copy_tensor_accessor_w_to_cpu_if_necessary(Z, cpu);
    expect(Zh.at<DataType::FLOAT>({3, 1}) == 16.0f && Zh.at<DataType::FLOAT>({0, 0}) == 42.0f, "ElementUnary scalar multiply");
  }
  // Transpose [4,2] -> [2,4]
  {
    TensorShape ts{TensorDims{{2, 4}}, DataType::FLOAT};
    GenericTensorAccessorW T = gpu.allocate_tensor(ts);
    Kernels::Transpose::forward_kernel(stream, TransposeAttrs{{1, 0}}, Y, T);
    GenericTensorAccessorW Th = copy_tensor_accessor_w(T, cpu);
    expect(Th.at<DataType::FLOAT>({1, 2}) == 9.5f && Th.at<DataType::FLOAT>({0, 3}) == 7.5f, "Transpose");
  }
  // Gather along dim 1 with an INT32 index
  {
    TensorShape is{TensorDims{{4, 1}}, DataType::INT32}, os{TensorDims{{4, 1}}, DataType::FLOAT};
    GenericTensorAccessorW Ih = cpu.allocate_tensor(is);
    for (int64_t i = 0; i < 4; i++) Ih.at<DataType::INT32>({i, 0}) = (int32_t)(i % 2);
    GenericTensorAccessorW I = copy_tensor_accessor_w(Ih, gpu);
    GenericTensorAccessorW O = gpu.allocate_tensor(os);
    std::optional<GatherPerDeviceState> gs = Kernels::Gather::init_kernel(DeviceType::GPU, handle, ff_dim_t{1});
    Kernels::Gather::forward_kernel(stream, gs, Y, I, O);
    GenericTensorAccessorW Oh = copy_tensor_accessor_w(O, cpu);
    expect(Oh.at<DataType::FLOAT>({0, 0}) == 21.0f && Oh.at<DataType::FLOAT>({1, 0}) == -1.0f &&
               Oh.at<DataType::FLOAT>({2, 0}) == 5.0f && Oh.at<DataType::FLOAT>({3, 0}) == 8.0f,
           "Gather");
  }
  static_assert(std::is_same_v<real_type_t<DataType::INT64>, int64_t>, "real_type_t");
  static_assert(type_to_data_type_enum_v<float> == DataType::FLOAT, "type_to_data_type_enum_v");
  ProfilingSettings settings{0, 1};
  (void)settings;
  return bad;
}
