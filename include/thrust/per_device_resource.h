// thrust::get_per_device_resource<MR>(system): the instance of MR that belongs to the current
// device of `system` (thrust/per_device_resource.h:34-97).  One process drives one GPU here, so
// it is the process-wide instance of MR; thrust::per_device_allocator draws from it.
#pragma once
#include <thrust/detail/execution_policy.h>
#include <thrust/mr/allocator.h>
#include <thrust/mr/memory_resource.h>

namespace thrust {
template <typename MR, typename D>
inline MR* get_per_device_resource(const thrust::detail::execution_policy_base<D>&) {
  return thrust::mr::get_global_resource<MR>();
}
template <typename T, typename MR, typename ExecutionPolicy>
class per_device_allocator : public thrust::mr::allocator<T, MR> {
 public:
  template <typename U> struct rebind { typedef per_device_allocator<U, MR, ExecutionPolicy> other; };
  per_device_allocator() : thrust::mr::allocator<T, MR>(get_per_device_resource<MR>(ExecutionPolicy())) {}
  template <typename U>
  per_device_allocator(const per_device_allocator<U, MR, ExecutionPolicy>& o) : thrust::mr::allocator<T, MR>(o) {}
};
}  // namespace thrust
