// Accessors, allocators, streams and handles of the host mirror, over the C ABI.
#include "ffk.h"
#include "kernels/accessor.h"
#include "kernels/allocation.h"
#include "kernels/device_stream_t.h"
#include <cstdlib>
#include <cstring>

namespace FlexFlow {

void check_ffk(int status, char const *what) {
  if (status != FFK_OK) {
    throw FatalError(std::string(what) + ": " + ffk_last_error());
  }
}

// ---- accessors ------------------------------------------------------------

int64_t calculate_accessor_offset(TensorDimsCoord const &coord, TensorDims const &dims) {
  if (coord.size() != dims.ff_ordered.size()) {
    throw std::runtime_error("Number of indices does not match the number of dimensions");
  }
  int64_t offset = 0, multiplier = 1;
  for (int i = (int)coord.size() - 1; i >= 0; i--) {
    if (coord[i] < 0 || coord[i] >= dims.ff_ordered[i]) {
      throw std::runtime_error("In dimension " + std::to_string(i) + ": index out of bounds");
    }
    offset += coord[i] * multiplier;
    multiplier *= dims.ff_ordered[i];
  }
  return offset;
}

GenericTensorAccessorR read_only_accessor_from_write_accessor(GenericTensorAccessorW const &w) {
  return GenericTensorAccessorR{w.shape, w.ptr, w.device_type};
}
TensorShape get_tensor_shape_for_accessor_r(GenericTensorAccessorR const &a) { return a.shape; }
TensorShape get_tensor_shape_for_accessor_w(GenericTensorAccessorW const &a) { return a.shape; }

void copy_accessor_data_to_l_from_r(GenericTensorAccessorW const &dst, GenericTensorAccessorR const &src) {
  if (dst.shape != src.shape) {
    throw std::runtime_error("copy_accessor_data_to_l_from_r: shapes differ");
  }
  size_t bytes = (size_t)get_size_in_bytes(dst.shape);
  bool dg = dst.device_type == DeviceType::GPU, sg = src.device_type == DeviceType::GPU;
  if (!dg && !sg) {
    memcpy(dst.ptr, src.ptr, bytes);
  } else {
    int kind = dg && sg ? FFK_D2D : (dg ? FFK_H2D : FFK_D2H);
    check_ffk(ffk_memcpy(dst.ptr, src.ptr, bytes, kind, nullptr), "ffk_memcpy");
  }
}

void fill_with_zeros(GenericTensorAccessorW const &a) {
  size_t bytes = (size_t)get_size_in_bytes(a.shape);
  if (a.device_type == DeviceType::CPU) {
    memset(a.ptr, 0, bytes);
  } else {
    check_ffk(ffk_fill_zero(a.ptr, bytes, nullptr), "ffk_fill_zero");
    check_ffk(ffk_stream_synchronize(nullptr), "ffk_stream_synchronize");
  }
}

// ---- allocators -----------------------------------------------------------

void *LocalCPUAllocator::allocate(size_t n) {
  void *p = malloc(n > 0 ? n : 1);
  if (p == nullptr) throw std::runtime_error("Failed to allocate host memory");
  ptrs.insert(p);
  return p;
}
void LocalCPUAllocator::deallocate(void *p) {
  if (ptrs.erase(p) == 0) throw std::runtime_error("Deallocating a pointer that was not allocated by this Allocator");
  free(p);
}
LocalCPUAllocator::~LocalCPUAllocator() {
  for (void *p : ptrs) free(p);
}

void *LocalCudaAllocator::allocate(size_t n) {
  void *p = nullptr;
  check_ffk(ffk_malloc(&p, n > 0 ? n : 1), "ffk_malloc");
  ptrs.insert(p);
  return p;
}
void LocalCudaAllocator::deallocate(void *p) {
  if (ptrs.erase(p) == 0) throw std::runtime_error("Deallocating a pointer that was not allocated by this Allocator");
  check_ffk(ffk_free(p), "ffk_free");
}
LocalCudaAllocator::~LocalCudaAllocator() {
  for (void *p : ptrs) ffk_free(p);
}

GenericTensorAccessorW Allocator::allocate_tensor(TensorShape const &s) {
  void *p = i_allocator->allocate((size_t)get_size_in_bytes(s));
  return GenericTensorAccessorW{s, p, i_allocator->get_allocation_device_type()};
}
void Allocator::deallocate_tensor(GenericTensorAccessorW const &t) {
  if (t.device_type != get_allocation_device_type()) throw std::runtime_error("deallocate_tensor: device type mismatch");
  i_allocator->deallocate(t.ptr);
}
void Allocator::deallocate_tensor(GenericTensorAccessorR const &t) {
  if (t.device_type != get_allocation_device_type()) throw std::runtime_error("deallocate_tensor: device type mismatch");
  i_allocator->deallocate(const_cast<void *>(t.ptr));
}
void *Allocator::allocate(size_t n) { return i_allocator->allocate(n); }
void Allocator::deallocate(void *p) { i_allocator->deallocate(p); }
DeviceType Allocator::get_allocation_device_type() const { return i_allocator->get_allocation_device_type(); }

Allocator create_local_cpu_memory_allocator() { return Allocator::create<LocalCPUAllocator>(); }
Allocator create_local_cuda_memory_allocator() { return Allocator::create<LocalCudaAllocator>(); }
Allocator create_local_allocator_for_device_type(DeviceType t) {
  return t == DeviceType::GPU ? create_local_cuda_memory_allocator() : create_local_cpu_memory_allocator();
}

GenericTensorAccessorW copy_tensor_accessor_w(GenericTensorAccessorW const &src, Allocator &allocator) {
  GenericTensorAccessorW dst = allocator.allocate_tensor(src.shape);
  copy_accessor_data_to_l_from_r(dst, read_only_accessor_from_write_accessor(src));
  return dst;
}
GenericTensorAccessorW copy_tensor_accessor_r(GenericTensorAccessorR const &src, Allocator &allocator) {
  GenericTensorAccessorW dst = allocator.allocate_tensor(src.shape);
  copy_accessor_data_to_l_from_r(dst, src);
  return dst;
}

// src/kernels/copy_tensor_accessor.cc: the source itself when it is host-resident already
GenericTensorAccessorR copy_tensor_accessor_r_to_cpu_if_necessary(GenericTensorAccessorR const &src, Allocator &cpu_allocator) {
  if (cpu_allocator.get_allocation_device_type() != DeviceType::CPU) {
    throw std::runtime_error("copy_tensor_accessor_r_to_cpu_if_necessary: a CPU allocator is required");
  }
  if (src.device_type == DeviceType::CPU) return src;
  return read_only_accessor_from_write_accessor(copy_tensor_accessor_r(src, cpu_allocator));
}
GenericTensorAccessorW copy_tensor_accessor_w_to_cpu_if_necessary(GenericTensorAccessorW const &src, Allocator &cpu_allocator) {
  if (cpu_allocator.get_allocation_device_type() != DeviceType::CPU) {
    throw std::runtime_error("copy_tensor_accessor_w_to_cpu_if_necessary: a CPU allocator is required");
  }
  if (src.device_type == DeviceType::CPU) return src;
  return copy_tensor_accessor_w(src, cpu_allocator);
}

// ---- streams and handles --------------------------------------------------

// One stream for the process's device work (the reference's get_legion_stream
// creates a new stream on every call, src/cuda/cuda_helper.cu:9-16).
static ffStream_t process_stream() {
  static ffStream_t s = [] {
    ffStream_t st = nullptr;
    check_ffk(ffk_stream_create(&st), "ffk_stream_create");
    return st;
  }();
  return s;
}

device_stream_t get_gpu_device_stream() { return device_stream_t::gpu(process_stream()); }
device_stream_t get_cpu_device_stream() { return device_stream_t::cpu(); }
device_stream_t get_stream_for_device_type(DeviceType t) {
  return t == DeviceType::GPU ? get_gpu_device_stream() : get_cpu_device_stream();
}

ManagedFFStream::ManagedFFStream() : stream(nullptr) {
  check_ffk(ffk_stream_create(&stream), "ffk_stream_create");
}
ManagedFFStream::ManagedFFStream(ManagedFFStream &&o) noexcept : stream(o.stream) { o.stream = nullptr; }
ManagedFFStream::~ManagedFFStream() {
  if (stream != nullptr) ffk_stream_destroy(stream);
}

ManagedPerDeviceFFHandle::ManagedPerDeviceFFHandle(size_t workSpaceSize, bool allowTensorOpMathConversion)
    : owns(true) {
  handle.dnn = nullptr;
  handle.blas = nullptr;
  handle.workSpace = nullptr;
  handle.workSpaceSize = workSpaceSize;
  handle.allowTensorOpMathConversion = allowTensorOpMathConversion;
  handle.stream = process_stream();
  check_ffk(ffk_malloc(&handle.workSpace, workSpaceSize), "ffk_malloc(workSpace)");
}
ManagedPerDeviceFFHandle::ManagedPerDeviceFFHandle(ManagedPerDeviceFFHandle &&o) noexcept
    : handle(o.handle), owns(o.owns) {
  o.owns = false;
}
ManagedPerDeviceFFHandle::~ManagedPerDeviceFFHandle() {
  if (owns) ffk_free(handle.workSpace);
}
ManagedPerDeviceFFHandle initialize_single_gpu_handle(size_t workSpaceSize, bool allowTensorOpMathConversion) {
  return ManagedPerDeviceFFHandle(workSpaceSize, allowTensorOpMathConversion);
}
device_handle_t device_handle_t_from_managed_ff_handle(ManagedPerDeviceFFHandle const &h) {
  return device_handle_t::for_gpu(h.raw_handle());
}

}  // namespace FlexFlow
