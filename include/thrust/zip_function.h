// thrust::zip_function / make_zip_function: turns a function of N arguments into a function of one
// N-tuple, so that a lambda written for the elements can be applied to what a zip_iterator yields
// (thrust/zip_function.h:38-180; testing/zip_function.cu).
#pragma once
#include <cstddef>
#include <utility>

#include <thrust/tuple.h>

namespace thrust {
namespace detail {
template <std::size_t... Is>
struct index_list {};
template <std::size_t N, std::size_t... Is>
struct make_index_list : make_index_list<N - 1, N - 1, Is...> {};
template <std::size_t... Is>
struct make_index_list<0, Is...> { typedef index_list<Is...> type; };

template <typename F, typename Tuple, std::size_t... Is>
__host__ __device__ auto apply_to_elements(F& f, Tuple&& t, index_list<Is...>)
    -> decltype(f(thrust::get<Is>(std::forward<Tuple>(t))...)) {
  return f(thrust::get<Is>(std::forward<Tuple>(t))...);
}
}  // namespace detail

template <typename F>
class zip_function {
 public:
  __host__ __device__ zip_function() : f_() {}
  __host__ __device__ zip_function(F f) : f_(f) {}
  template <typename Tuple>
  __host__ __device__ auto operator()(Tuple&& t) const -> decltype(detail::apply_to_elements(
      std::declval<F&>(), std::forward<Tuple>(t),
      typename detail::make_index_list<thrust::tuple_size<typename std::decay<Tuple>::type>::value>::type())) {
    return detail::apply_to_elements(
        f_, std::forward<Tuple>(t),
        typename detail::make_index_list<thrust::tuple_size<typename std::decay<Tuple>::type>::value>::type());
  }

 private:
  mutable F f_;
};
template <typename F>
__host__ __device__ zip_function<typename std::decay<F>::type> make_zip_function(F&& f) {
  return zip_function<typename std::decay<F>::type>(std::forward<F>(f));
}

}  // namespace thrust
