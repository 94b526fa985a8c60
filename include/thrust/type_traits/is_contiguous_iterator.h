// thrust::is_contiguous_iterator<It>: does the range lie in one array, so that its address is all
// an algorithm needs (thrust/type_traits/is_contiguous_iterator.h:40-230)?  Pointers, device_ptr
// and the iterators of std::vector / host_vector do; computed iterators do not.
#pragma once
#include <type_traits>
#include <vector>

#include <thrust/device_ptr.h>
#include <thrust/iterator/iterator_traits.h>

namespace thrust {
namespace detail {
template <typename It, typename = void>
struct is_vector_iterator : std::false_type {};
template <typename It>
struct is_vector_iterator<It, typename std::enable_if<!std::is_pointer<It>::value && !std::is_same<typename std::iterator_traits<It>::value_type, bool>::value &&
                                                      (std::is_same<It, typename std::vector<typename std::iterator_traits<It>::value_type>::iterator>::value ||
                                                       std::is_same<It, typename std::vector<typename std::iterator_traits<It>::value_type>::const_iterator>::value)>::type>
    : std::true_type {};
}  // namespace detail
template <typename It>
struct is_contiguous_iterator
    : std::integral_constant<bool, std::is_pointer<It>::value || thrust::detail::is_device_iterator<It>::value ||
                                       thrust::detail::is_vector_iterator<It>::value> {};
template <typename It>
constexpr bool is_contiguous_iterator_v = is_contiguous_iterator<It>::value;
}  // namespace thrust
