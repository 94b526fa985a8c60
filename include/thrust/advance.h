// thrust::advance: moves an iterator by n positions (thrust/advance.h, thrust/system/detail/generic/advance.inl).
#pragma once
#include <iterator>

namespace thrust {
template <typename It, typename Distance>
inline void advance(It& it, Distance n) {
  std::advance(it, n);
}
}  // namespace thrust
