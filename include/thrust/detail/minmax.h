// thrust::min, thrust::max: of two values, with operator< or the caller's order; the first
// argument when neither comes before the other (thrust/detail/minmax.h:24-54 of the reference,
// reached through thrust/extrema.h and thrust/functional.h).
#pragma once
#include <thrust/detail/config.h>

namespace thrust {
template <typename T, typename Comp>
__host__ __device__ inline T min THRUST_AMD_NO_MACRO(const T& a, const T& b, Comp comp) { return comp(b, a) ? b : a; }
template <typename T>
__host__ __device__ inline T min THRUST_AMD_NO_MACRO(const T& a, const T& b) { return b < a ? b : a; }
template <typename T, typename Comp>
__host__ __device__ inline T max THRUST_AMD_NO_MACRO(const T& a, const T& b, Comp comp) { return comp(a, b) ? b : a; }
template <typename T>
__host__ __device__ inline T max THRUST_AMD_NO_MACRO(const T& a, const T& b) { return a < b ? b : a; }
}  // namespace thrust
