// Allocator / IAllocator and the local CPU / device allocators (reference:
// lib/kernels/include/kernels/allocation.h:10-42, local_cpu_allocator.h,
// local_cuda_allocator.h, create_local_allocator_for_device_type.h,
// copy_tensor_accessor.h; bodies lib/kernels/src/kernels/local_*_allocator.cc).
// Headers under those reference names include this one.  The device allocator
// keeps the reference's name so callers compile unchanged.
#pragma once
#include "kernels/accessor.h"
#include <cstddef>
#include <memory>
#include <unordered_set>

namespace FlexFlow {

struct IAllocator {
  virtual void *allocate(size_t) = 0;
  virtual void deallocate(void *) = 0;
  virtual DeviceType get_allocation_device_type() const = 0;
  virtual ~IAllocator() = default;
};

struct Allocator {
  Allocator() = delete;
  explicit Allocator(std::shared_ptr<IAllocator> ptr) : i_allocator(std::move(ptr)) {}

  GenericTensorAccessorW allocate_tensor(TensorShape const &tensor_shape);
  void deallocate_tensor(GenericTensorAccessorW const &);
  void deallocate_tensor(GenericTensorAccessorR const &);
  void *allocate(size_t mem_size);
  void deallocate(void *ptr);
  DeviceType get_allocation_device_type() const;

  template <typename T, typename... Args>
  static Allocator create(Args &&...args) {
    return Allocator(std::make_shared<T>(std::forward<Args>(args)...));
  }

 private:
  std::shared_ptr<IAllocator> i_allocator;
};

// Both free everything still allocated when destroyed; deallocating a pointer
// they do not own throws (the reference asserts, local_cpu_allocator.cc:15-20).
struct LocalCPUAllocator : IAllocator {
  void *allocate(size_t) override;
  void deallocate(void *) override;
  DeviceType get_allocation_device_type() const override { return DeviceType::CPU; }
  ~LocalCPUAllocator() override;
 private:
  std::unordered_set<void *> ptrs;
};

struct LocalCudaAllocator : IAllocator {
  void *allocate(size_t) override;
  void deallocate(void *) override;
  DeviceType get_allocation_device_type() const override { return DeviceType::GPU; }
  ~LocalCudaAllocator() override;
 private:
  std::unordered_set<void *> ptrs;
};

Allocator create_local_cpu_memory_allocator();
Allocator create_local_cuda_memory_allocator();
Allocator create_local_allocator_for_device_type(DeviceType);

// copy_tensor_accessor.h:9-25: a fresh tensor from the allocator with the source's contents
// (whatever side each lives on); the _to_cpu_if_necessary forms return the source itself when
// it already is host-resident.
GenericTensorAccessorW copy_tensor_accessor_w(GenericTensorAccessorW const &src, Allocator &allocator);
GenericTensorAccessorW copy_tensor_accessor_r(GenericTensorAccessorR const &src, Allocator &allocator);
GenericTensorAccessorR copy_tensor_accessor_r_to_cpu_if_necessary(GenericTensorAccessorR const &, Allocator &cpu_allocator);
GenericTensorAccessorW copy_tensor_accessor_w_to_cpu_if_necessary(GenericTensorAccessorW const &, Allocator &cpu_allocator);

}  // namespace FlexFlow
