// Function objects of the front end.  For the device system these types are also
// dispatch keys: the C ABI knows a closed set of operators, and an algorithm reaches
// its kernel when the functor type is one of the recognised ones below (the reference
// applies the same idea to sorting, where only exactly less<Key> / greater<Key> take
// the radix path, thrust/system/cuda/detail/sort.h:1518-1523).
//   binary operators   plus, minimum, maximum            (reduce, scans, reduce_by_key)
//   orderings          less, greater                     (sort, merge)
//   equivalence        equal_to                          (unique, reduce_by_key)
//   unary predicates   placeholder comparisons (_1 < t), identity / "is true",
//                      logical_not                       (copy_if, partition, remove_if, count_if)
//   unary transforms   identity, negate, square          (transform_reduce, transform scans)
#pragma once
#include <thrust/detail/config.h>
#include <thrust/detail/minmax.h>
#include <thrust/detail/placeholder_expressions.h>

namespace thrust {

template <typename A, typename R> struct unary_function { typedef A argument_type; typedef R result_type; };
template <typename A1, typename A2, typename R>
struct binary_function { typedef A1 first_argument_type; typedef A2 second_argument_type; typedef R result_type; };

#define THRUST_AMD_BINARY_FUNCTOR(NAME, RESULT, EXPR)                                   \
  template <typename T = void>                                                          \
  struct NAME {                                                                         \
    typedef T first_argument_type;                                                      \
    typedef T second_argument_type;                                                     \
    typedef RESULT result_type;                                                         \
    constexpr RESULT operator()(const T& lhs, const T& rhs) const { return EXPR; }      \
  };                                                                                    \
  template <>                                                                           \
  struct NAME<void> {                                                                   \
    template <typename A, typename B>                                                   \
    constexpr auto operator()(const A& lhs, const B& rhs) const -> decltype(EXPR) { return EXPR; } \
  };

THRUST_AMD_BINARY_FUNCTOR(plus, T, lhs + rhs)
THRUST_AMD_BINARY_FUNCTOR(minus, T, lhs - rhs)
THRUST_AMD_BINARY_FUNCTOR(multiplies, T, lhs * rhs)
THRUST_AMD_BINARY_FUNCTOR(divides, T, lhs / rhs)
THRUST_AMD_BINARY_FUNCTOR(modulus, T, lhs % rhs)
THRUST_AMD_BINARY_FUNCTOR(bit_and, T, lhs & rhs)
THRUST_AMD_BINARY_FUNCTOR(bit_or, T, lhs | rhs)
THRUST_AMD_BINARY_FUNCTOR(bit_xor, T, lhs ^ rhs)
THRUST_AMD_BINARY_FUNCTOR(logical_and, bool, lhs && rhs)
THRUST_AMD_BINARY_FUNCTOR(logical_or, bool, lhs || rhs)
THRUST_AMD_BINARY_FUNCTOR(equal_to, bool, lhs == rhs)
THRUST_AMD_BINARY_FUNCTOR(not_equal_to, bool, lhs != rhs)
THRUST_AMD_BINARY_FUNCTOR(less, bool, lhs < rhs)
THRUST_AMD_BINARY_FUNCTOR(greater, bool, lhs > rhs)
THRUST_AMD_BINARY_FUNCTOR(less_equal, bool, lhs <= rhs)
THRUST_AMD_BINARY_FUNCTOR(greater_equal, bool, lhs >= rhs)
THRUST_AMD_BINARY_FUNCTOR(maximum, T, (lhs < rhs ? rhs : lhs))
THRUST_AMD_BINARY_FUNCTOR(minimum, T, (lhs < rhs ? lhs : rhs))
#undef THRUST_AMD_BINARY_FUNCTOR

template <typename T = void>
struct identity {
  typedef T argument_type;
  typedef T result_type;
  constexpr const T& operator()(const T& x) const { return x; }
};
template <>
struct identity<void> {
  template <typename A>
  constexpr const A& operator()(const A& x) const { return x; }
};

template <typename T = void>
struct logical_not {
  typedef T argument_type;
  typedef bool result_type;
  constexpr bool operator()(const T& x) const { return !x; }
};
template <>
struct logical_not<void> {
  template <typename A>
  constexpr bool operator()(const A& x) const { return !x; }
};
// project1st / project2nd return one of their two arguments (thrust/functional.h:1307-1401 in
// the reference); not1 / not2 negate a predicate (thrust/functional.h:1407-1493).
template <typename T1 = void, typename T2 = void>
struct project1st {
  typedef T1 first_argument_type;
  typedef T2 second_argument_type;
  typedef T1 result_type;
  constexpr const T1& operator()(const T1& lhs, const T2&) const { return lhs; }
};
template <>
struct project1st<void, void> {
  template <typename A, typename B>
  constexpr const A& operator()(const A& lhs, const B&) const { return lhs; }
};
template <typename T1 = void, typename T2 = void>
struct project2nd {
  typedef T1 first_argument_type;
  typedef T2 second_argument_type;
  typedef T2 result_type;
  constexpr const T2& operator()(const T1&, const T2& rhs) const { return rhs; }
};
template <>
struct project2nd<void, void> {
  template <typename A, typename B>
  constexpr const B& operator()(const A&, const B& rhs) const { return rhs; }
};
template <typename Predicate>
struct unary_negate {
  typedef bool result_type;
  Predicate pred;
  explicit constexpr unary_negate(const Predicate& p) : pred(p) {}
  template <typename A>
  constexpr bool operator()(const A& x) const { return !pred(x); }
};
template <typename Predicate>
constexpr unary_negate<Predicate> not1(const Predicate& pred) { return unary_negate<Predicate>(pred); }
template <typename Predicate>
struct binary_negate {
  typedef bool result_type;
  Predicate pred;
  explicit constexpr binary_negate(const Predicate& p) : pred(p) {}
  template <typename A, typename B>
  constexpr bool operator()(const A& x, const B& y) const { return !pred(x, y); }
};
template <typename Predicate>
constexpr binary_negate<Predicate> not2(const Predicate& pred) { return binary_negate<Predicate>(pred); }

template <typename T = void>
struct negate {
  typedef T argument_type;
  typedef T result_type;
  constexpr T operator()(const T& x) const { return -x; }
};

template <typename T = void>
struct square {
  typedef T argument_type;
  typedef T result_type;
  constexpr T operator()(const T& x) const { return x * x; }
};
template <>
struct negate<void> {
  template <typename A>
  constexpr auto operator()(const A& x) const -> decltype(-x) { return -x; }
};
template <>
struct square<void> {
  template <typename A>
  constexpr auto operator()(const A& x) const -> decltype(x * x) { return x * x; }
};

namespace detail {
// `x CMP value` as a unary predicate; CMP is a thrust_amd_cmp code (0 LT .. 5 NE).  It is what
// `_1 CMP value` builds: the one placeholder expression the library's own selection kernels
// take (as a comparison code and a threshold), and a node like any other inside larger
// expressions (`_1 > 2 && _1 < 9`).
#if defined(__GNUC__)
#pragma GCC diagnostic push
#pragma GCC diagnostic ignored "-Wsign-compare"  // the expression is the caller's, conversions included
#endif
template <int CMP, typename T>
struct compare_with : lambda::actor_base {
  T value;
  constexpr explicit compare_with(const T& v) : value(v) {}
  // evaluated on the argument as it is, under the usual arithmetic conversions, as the
  // reference's placeholder expression `_1 < t` does (further arguments are ignored)
  template <typename A, typename... Rest>
  constexpr bool operator()(const A& x, Rest&&...) const {
    return CMP == 0 ? x < value : CMP == 1 ? x <= value : CMP == 2 ? x > value
         : CMP == 3 ? x >= value : CMP == 4 ? x == value : x != value;
  }
};
#if defined(__GNUC__)
#pragma GCC diagnostic pop
#endif

namespace lambda {
// `_1 CMP value` and `value CMP _1` with a plain value (more specialised than the general
// operators of placeholder_expressions.h, so these are chosen)
#define THRUST_AMD_PLACEHOLDER_CMP(OP, CODE, SWAPPED)                                                  \
  template <typename T, typename = typename std::enable_if<!is_actor<T>::value>::type>                 \
  constexpr compare_with<CODE, T> operator OP(argument<0>, const T& v) { return compare_with<CODE, T>(v); } \
  template <typename T, typename = typename std::enable_if<!is_actor<T>::value>::type>                 \
  constexpr compare_with<SWAPPED, T> operator OP(const T& v, argument<0>) { return compare_with<SWAPPED, T>(v); }
THRUST_AMD_PLACEHOLDER_CMP(<, 0, 2)
THRUST_AMD_PLACEHOLDER_CMP(<=, 1, 3)
THRUST_AMD_PLACEHOLDER_CMP(>, 2, 0)
THRUST_AMD_PLACEHOLDER_CMP(>=, 3, 1)
THRUST_AMD_PLACEHOLDER_CMP(==, 4, 4)
THRUST_AMD_PLACEHOLDER_CMP(!=, 5, 5)
#undef THRUST_AMD_PLACEHOLDER_CMP
}  // namespace lambda
}  // namespace detail

// thrust::placeholders::_1 .. _10 (thrust/functional.h:1430-1520 of the reference)
namespace placeholders {
static const thrust::detail::lambda::argument<0> _1 = {};
static const thrust::detail::lambda::argument<1> _2 = {};
static const thrust::detail::lambda::argument<2> _3 = {};
static const thrust::detail::lambda::argument<3> _4 = {};
static const thrust::detail::lambda::argument<4> _5 = {};
static const thrust::detail::lambda::argument<5> _6 = {};
static const thrust::detail::lambda::argument<6> _7 = {};
static const thrust::detail::lambda::argument<7> _8 = {};
static const thrust::detail::lambda::argument<8> _9 = {};
static const thrust::detail::lambda::argument<9> _10 = {};
}  // namespace placeholders

}  // namespace thrust
