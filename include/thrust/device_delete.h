// thrust::device_delete: the counterpart of device_new (thrust/device_delete.h,
// thrust/detail/device_delete.inl: destroy_range + device_free; the element types of the device
// system have trivial destructors, so freeing is all there is to do).
#pragma once
#include <cstddef>

#include <thrust/device_ptr.h>

namespace thrust {

template <typename T>
inline void device_delete(device_ptr<T> p, const std::size_t = 1) {
  thrust::device_free(p);
}

}  // namespace thrust
