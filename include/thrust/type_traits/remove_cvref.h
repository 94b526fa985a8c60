// thrust::remove_cvref, remove_cvref_t (thrust/type_traits/remove_cvref.h:25-50).
#pragma once
#include <type_traits>

namespace thrust {
template <typename T>
struct remove_cvref { typedef typename std::remove_cv<typename std::remove_reference<T>::type>::type type; };
template <typename T>
using remove_cvref_t = typename remove_cvref<T>::type;
}  // namespace thrust
