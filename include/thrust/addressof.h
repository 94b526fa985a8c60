// thrust::addressof: the address of an object whatever its operator& does (thrust/addressof.h).
#pragma once
#include <memory>

#include <thrust/detail/config.h>

namespace thrust {
template <typename T>
__host__ __device__ inline T* addressof(T& arg) {
  return reinterpret_cast<T*>(&const_cast<char&>(reinterpret_cast<const volatile char&>(arg)));
}
}  // namespace thrust
