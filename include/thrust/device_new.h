// thrust::device_new: n objects of T in device memory, copies of T() or of a given value; into
// memory the caller has (placement) or freshly allocated (thrust/device_new.h,
// thrust/detail/device_new.inl:30-60: device_malloc + uninitialized_fill).
#pragma once
#include <cstddef>

#include <thrust/device_ptr.h>
#include <thrust/uninitialized_fill.h>

namespace thrust {

template <typename T>
device_ptr<T> device_new(device_ptr<void> p, const T& exemplar, const std::size_t n = 1) {
  device_ptr<T> result(static_cast<T*>(p.get()));
  thrust::uninitialized_fill(result, result + n, exemplar);
  return result;
}
template <typename T>
device_ptr<T> device_new(device_ptr<void> p, const std::size_t n = 1) {
  return thrust::device_new<T>(p, T(), n);
}
template <typename T>
device_ptr<T> device_new(const std::size_t n = 1) {
  return thrust::device_new<T>(thrust::device_malloc(n * sizeof(T)), n);
}

}  // namespace thrust
