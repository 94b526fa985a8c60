// thrust::is_execution_policy<T> (thrust/type_traits/is_execution_policy.h:30-50).
#pragma once
#include <type_traits>

#include <thrust/iterator/iterator_traits.h>

namespace thrust {
template <typename T>
struct is_execution_policy : thrust::detail::is_execution_policy<typename std::decay<T>::type> {};
template <typename T>
constexpr bool is_execution_policy_v = is_execution_policy<T>::value;
}  // namespace thrust
