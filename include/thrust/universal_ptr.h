// thrust::universal_ptr<T>: a pointer into storage that host code and kernels both address
// (thrust/universal_ptr.h:24-30).  Such storage is handed out as device_ptr here
// (thrust/universal_vector.h of this tree), so the name is an alias.
#pragma once
#include <thrust/device_ptr.h>

namespace thrust {
template <typename T>
using universal_ptr = thrust::device_ptr<T>;
}  // namespace thrust
