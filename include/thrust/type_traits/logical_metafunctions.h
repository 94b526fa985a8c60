// thrust::conjunction, disjunction, negation and their _value forms
// (thrust/type_traits/logical_metafunctions.h:30-180): the standard's, under this namespace.
#pragma once
#include <type_traits>

namespace thrust {
using std::conjunction;
using std::disjunction;
using std::negation;
template <typename... Ts>
constexpr bool conjunction_v = conjunction<Ts...>::value;
template <typename... Ts>
constexpr bool disjunction_v = disjunction<Ts...>::value;
template <typename T>
constexpr bool negation_v = negation<T>::value;
template <bool... Bs>
struct conjunction_value : std::integral_constant<bool, (Bs && ...)> {};
template <bool... Bs>
struct disjunction_value : std::integral_constant<bool, (Bs || ...)> {};
template <bool B>
struct negation_value : std::integral_constant<bool, !B> {};
}  // namespace thrust
