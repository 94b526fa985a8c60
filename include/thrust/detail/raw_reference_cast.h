// thrust::raw_reference_cast: the plain reference behind a device_reference
// (thrust/detail/raw_reference_cast.h:150-190).  What it returns names device memory: code that
// runs on the device may use it, the host may only take its address.  A plain reference, which
// is what dereferencing yields inside a kernel, passes through unchanged.
#pragma once
#include <thrust/device_ptr.h>

namespace thrust {
template <typename T>
__host__ __device__ inline T& raw_reference_cast(T& ref) { return ref; }
template <typename T>
__host__ __device__ inline const T& raw_reference_cast(const T& ref) { return ref; }
template <typename T>
__host__ __device__ inline T& raw_reference_cast(const device_reference<T>& ref) { return *(&ref).get(); }
template <typename T>
__host__ __device__ inline T& raw_reference_cast(device_reference<T>& ref) { return *(&ref).get(); }
}  // namespace thrust
