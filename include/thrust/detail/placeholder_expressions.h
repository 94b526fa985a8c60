// Placeholder expressions: `_1 * _2 + 1.0f`, `a * _1 + _2`, `_1 += _2`, `-_1`, `_1 < _2` ... build
// small function objects, the reference's thrust::placeholders
// (thrust/functional.h:1430-1520 over thrust/detail/functional/actor.h and operators.h).
// An expression is a tree of three kinds of node, each callable with the arguments of the call:
//   argument<I>     yields argument I as it was passed (an lvalue stays an lvalue, so `_1 += _2`
//                   writes through it)
//   constant<T>     yields a value captured when the expression was built
//   unary / binary  apply an operator to what their operands yield
// Everything is __host__ __device__ and trivially copyable when the captured values are, so an
// expression travels into a kernel by value like any other functor (translation units compiled
// with hipcc).  The one shape the library's own kernels know without that, `_1 CMP value`,
// keeps its dedicated type (thrust::detail::compare_with, defined in thrust/functional.h).
#pragma once
#include <type_traits>
#include <utility>

#include <thrust/detail/config.h>

namespace thrust {
namespace detail {
namespace lambda {

struct actor_base {};
template <typename E>
struct is_actor : std::is_base_of<actor_base, typename std::decay<E>::type> {};

template <int I>
struct pick_argument {
  template <typename A0, typename... A>
  __host__ __device__ static constexpr auto from(A0&&, A&&... rest)
      -> decltype(pick_argument<I - 1>::from(static_cast<A&&>(rest)...)) {
    return pick_argument<I - 1>::from(static_cast<A&&>(rest)...);
  }
};
template <>
struct pick_argument<0> {
  template <typename A0, typename... A>
  __host__ __device__ static constexpr A0&& from(A0&& first, A&&...) { return static_cast<A0&&>(first); }
};

template <typename T>
struct constant : actor_base {
  T value;
  __host__ __device__ constexpr explicit constant(const T& v) : value(v) {}
  template <typename... A>
  __host__ __device__ constexpr const T& operator()(A&&...) const { return value; }
};

template <typename Op, typename X>
struct unary_expr : actor_base {
  X x;
  __host__ __device__ constexpr explicit unary_expr(const X& operand) : x(operand) {}
  template <typename... A>
  __host__ __device__ constexpr auto operator()(A&&... a) const -> decltype(Op::apply(std::declval<const X&>()(a...))) {
    return Op::apply(x(a...));
  }
};
template <typename Op, typename L, typename R>
struct binary_expr : actor_base {
  L l;
  R r;
  __host__ __device__ constexpr binary_expr(const L& left, const R& right) : l(left), r(right) {}
  template <typename... A>
  __host__ __device__ constexpr auto operator()(A&&... a) const
      -> decltype(Op::apply(std::declval<const L&>()(a...), std::declval<const R&>()(a...))) {
    return Op::apply(l(a...), r(a...));
  }
};

// an operand as a node: expressions as they are, anything else captured by value
template <typename T, bool = is_actor<T>::value>
struct as_node { typedef typename std::decay<T>::type type; };
template <typename T>
struct as_node<T, false> { typedef constant<typename std::decay<T>::type> type; };
template <typename T>
__host__ __device__ constexpr typename std::enable_if<is_actor<T>::value, const T&>::type node(const T& t) { return t; }
template <typename T>
__host__ __device__ constexpr typename std::enable_if<!is_actor<T>::value, constant<T> >::type node(const T& t) {
  return constant<T>(t);
}

struct op_assign {
  template <typename X, typename Y>
  __host__ __device__ static constexpr auto apply(X&& x, Y&& y) -> decltype(static_cast<X&&>(x) = static_cast<Y&&>(y)) {
    return static_cast<X&&>(x) = static_cast<Y&&>(y);
  }
};

template <int I>
struct argument : actor_base {
  template <typename... A>
  __host__ __device__ constexpr auto operator()(A&&... a) const -> decltype(pick_argument<I>::from(static_cast<A&&>(a)...)) {
    return pick_argument<I>::from(static_cast<A&&>(a)...);
  }
  // _1 = expression
  template <typename R>
  __host__ __device__ constexpr binary_expr<op_assign, argument, typename as_node<R>::type> operator=(const R& r) const {
    return binary_expr<op_assign, argument, typename as_node<R>::type>(*this, node(r));
  }
};

#define THRUST_AMD_LAMBDA_BINARY(NAME, OP)                                                                       \
  struct NAME {                                                                                                  \
    template <typename X, typename Y>                                                                            \
    __host__ __device__ static constexpr auto apply(X&& x, Y&& y)                                                \
        -> decltype(static_cast<X&&>(x) OP static_cast<Y&&>(y)) {                                                \
      return static_cast<X&&>(x) OP static_cast<Y&&>(y);                                                         \
    }                                                                                                            \
  };                                                                                                             \
  template <typename L, typename R,                                                                              \
            typename = typename std::enable_if<is_actor<L>::value || is_actor<R>::value>::type>                  \
  __host__ __device__ constexpr binary_expr<NAME, typename as_node<L>::type, typename as_node<R>::type>          \
  operator OP(const L& l, const R& r) {                                                                          \
    return binary_expr<NAME, typename as_node<L>::type, typename as_node<R>::type>(node(l), node(r));            \
  }
THRUST_AMD_LAMBDA_BINARY(op_plus, +)
THRUST_AMD_LAMBDA_BINARY(op_minus, -)
THRUST_AMD_LAMBDA_BINARY(op_multiplies, *)
THRUST_AMD_LAMBDA_BINARY(op_divides, /)
THRUST_AMD_LAMBDA_BINARY(op_modulus, %)
THRUST_AMD_LAMBDA_BINARY(op_bit_and, &)
THRUST_AMD_LAMBDA_BINARY(op_bit_or, |)
THRUST_AMD_LAMBDA_BINARY(op_bit_xor, ^)
THRUST_AMD_LAMBDA_BINARY(op_shift_left, <<)
THRUST_AMD_LAMBDA_BINARY(op_shift_right, >>)
THRUST_AMD_LAMBDA_BINARY(op_logical_and, &&)
THRUST_AMD_LAMBDA_BINARY(op_logical_or, ||)
THRUST_AMD_LAMBDA_BINARY(op_equal_to, ==)
THRUST_AMD_LAMBDA_BINARY(op_not_equal_to, !=)
THRUST_AMD_LAMBDA_BINARY(op_less, <)
THRUST_AMD_LAMBDA_BINARY(op_greater, >)
THRUST_AMD_LAMBDA_BINARY(op_less_equal, <=)
THRUST_AMD_LAMBDA_BINARY(op_greater_equal, >=)
THRUST_AMD_LAMBDA_BINARY(op_plus_assign, +=)
THRUST_AMD_LAMBDA_BINARY(op_minus_assign, -=)
THRUST_AMD_LAMBDA_BINARY(op_multiplies_assign, *=)
THRUST_AMD_LAMBDA_BINARY(op_divides_assign, /=)
THRUST_AMD_LAMBDA_BINARY(op_modulus_assign, %=)
THRUST_AMD_LAMBDA_BINARY(op_bit_and_assign, &=)
THRUST_AMD_LAMBDA_BINARY(op_bit_or_assign, |=)
THRUST_AMD_LAMBDA_BINARY(op_bit_xor_assign, ^=)
THRUST_AMD_LAMBDA_BINARY(op_shift_left_assign, <<=)
THRUST_AMD_LAMBDA_BINARY(op_shift_right_assign, >>=)
#undef THRUST_AMD_LAMBDA_BINARY

#define THRUST_AMD_LAMBDA_PREFIX(NAME, OP)                                                                       \
  struct NAME {                                                                                                  \
    template <typename X>                                                                                        \
    __host__ __device__ static constexpr auto apply(X&& x) -> decltype(OP static_cast<X&&>(x)) {                 \
      return OP static_cast<X&&>(x);                                                                             \
    }                                                                                                            \
  };                                                                                                             \
  template <typename X, typename = typename std::enable_if<is_actor<X>::value>::type>                            \
  __host__ __device__ constexpr unary_expr<NAME, X> operator OP(const X& x) {                                    \
    return unary_expr<NAME, X>(x);                                                                               \
  }
THRUST_AMD_LAMBDA_PREFIX(op_unary_plus, +)
THRUST_AMD_LAMBDA_PREFIX(op_negate, -)
THRUST_AMD_LAMBDA_PREFIX(op_logical_not, !)
THRUST_AMD_LAMBDA_PREFIX(op_bit_not, ~)
THRUST_AMD_LAMBDA_PREFIX(op_prefix_increment, ++)
THRUST_AMD_LAMBDA_PREFIX(op_prefix_decrement, --)
#undef THRUST_AMD_LAMBDA_PREFIX

#define THRUST_AMD_LAMBDA_SUFFIX(NAME, OP)                                                                       \
  struct NAME {                                                                                                  \
    template <typename X>                                                                                        \
    __host__ __device__ static constexpr auto apply(X&& x) -> decltype(static_cast<X&&>(x) OP) {                 \
      return static_cast<X&&>(x) OP;                                                                             \
    }                                                                                                            \
  };                                                                                                             \
  template <typename X, typename = typename std::enable_if<is_actor<X>::value>::type>                            \
  __host__ __device__ constexpr unary_expr<NAME, X> operator OP(const X& x, int) {                               \
    return unary_expr<NAME, X>(x);                                                                               \
  }
THRUST_AMD_LAMBDA_SUFFIX(op_suffix_increment, ++)
THRUST_AMD_LAMBDA_SUFFIX(op_suffix_decrement, --)
#undef THRUST_AMD_LAMBDA_SUFFIX

}  // namespace lambda
}  // namespace detail
}  // namespace thrust
