// thrust::pair / thrust::make_pair (return type of the *_by_key and partition_copy algorithms;
// usable in device code: the distributions of thrust::random keep their parameters in one).
#pragma once
#include <utility>

#include <thrust/detail/config.h>

namespace thrust {

template <typename T1, typename T2>
struct pair {
  typedef T1 first_type;
  typedef T2 second_type;
  T1 first;
  T2 second;
  __host__ __device__ pair() : first(), second() {}
  __host__ __device__ pair(const T1& a, const T2& b) : first(a), second(b) {}
  template <typename U1, typename U2>
  __host__ __device__ pair(const pair<U1, U2>& p) : first(p.first), second(p.second) {}
  template <typename U1, typename U2>
  pair(const std::pair<U1, U2>& p) : first(p.first), second(p.second) {}
};

template <typename T1, typename T2>
__host__ __device__ inline bool operator==(const pair<T1, T2>& a, const pair<T1, T2>& b) {
  return a.first == b.first && a.second == b.second;
}
template <typename T1, typename T2>
__host__ __device__ inline bool operator!=(const pair<T1, T2>& a, const pair<T1, T2>& b) { return !(a == b); }
template <typename T1, typename T2>
__host__ __device__ inline bool operator<(const pair<T1, T2>& a, const pair<T1, T2>& b) {
  return a.first < b.first || (!(b.first < a.first) && a.second < b.second);
}

template <typename T1, typename T2>
__host__ __device__ inline pair<T1, T2> make_pair(T1 a, T2 b) { return pair<T1, T2>(a, b); }

}  // namespace thrust
