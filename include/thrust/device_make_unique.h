// thrust::device_make_unique<T>(args...): one T in device memory, a copy of T(args...) built on
// the host, owned by a std::unique_ptr that gives the storage back to thrust::device_allocator
// (thrust/device_make_unique.h:40-58; testing/async_reduce_into.cu:383 uses it for result slots).
#pragma once
#include <utility>

#include <thrust/allocate_unique.h>
#include <thrust/device_allocator.h>
#include <thrust/device_new.h>
#include <thrust/device_ptr.h>

namespace thrust {
template <typename T, typename... Args>
inline auto device_make_unique(Args&&... args) -> decltype(uninitialized_allocate_unique<T>(device_allocator<T>())) {
  auto p = uninitialized_allocate_unique<T>(device_allocator<T>());
  device_new<T>(thrust::device_ptr<void>(p.get().get()), T(std::forward<Args>(args)...));
  return p;
}
}  // namespace thrust
