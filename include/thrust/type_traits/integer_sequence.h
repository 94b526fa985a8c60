// thrust::integer_sequence, index_sequence and their makers
// (thrust/type_traits/integer_sequence.h:35-90): the standard's, under this namespace.
#pragma once
#include <cstddef>
#include <utility>

namespace thrust {
template <typename T, T... Is>
using integer_sequence = std::integer_sequence<T, Is...>;
template <std::size_t... Is>
using index_sequence = std::index_sequence<Is...>;
template <typename T, T N>
using make_integer_sequence = std::make_integer_sequence<T, N>;
template <std::size_t N>
using make_index_sequence = std::make_index_sequence<N>;
}  // namespace thrust
