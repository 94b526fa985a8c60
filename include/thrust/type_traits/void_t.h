// thrust::void_t, thrust::voider (thrust/type_traits/void_t.h:25-55).
#pragma once
#include <type_traits>

namespace thrust {
template <typename...>
struct voider { typedef void type; };
template <typename... Ts>
using void_t = typename voider<Ts...>::type;
}  // namespace thrust
