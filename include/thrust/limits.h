// thrust::numeric_limits (thrust/limits.h: the standard's).
#pragma once
#include <limits>

namespace thrust {
template <typename T>
struct numeric_limits : std::numeric_limits<T> {};
}  // namespace thrust
