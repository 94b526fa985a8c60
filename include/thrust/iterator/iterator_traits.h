// iterator_value / iterator_system / contiguous-range helpers used by the dispatch layer.
#pragma once
#include <iterator>
#include <type_traits>
#include <vector>

#include <thrust/device_ptr.h>

namespace thrust {

// thrust::iterator_traits: std::iterator_traits unless a user specialises it for an iterator
// type of their own (the reference's tests do so for iterators that only define what an
// algorithm needs, testing/scan.cu:586-594).
template <typename It>
struct iterator_traits : std::iterator_traits<It> {};

namespace detail {
template <typename Traits, typename = void>
struct difference_of { typedef std::ptrdiff_t type; };
template <typename Traits>
struct difference_of<Traits, typename std::enable_if<!std::is_void<typename Traits::difference_type>::value>::type> {
  typedef typename Traits::difference_type type;
};
}  // namespace detail

template <typename It>
struct iterator_value { typedef typename thrust::iterator_traits<It>::value_type type; };
template <typename It>
struct iterator_difference { typedef typename detail::difference_of<thrust::iterator_traits<It> >::type type; };
namespace detail {
// The element type an algorithm hands to an output iterator: the iterator's own, or, for an
// iterator that names none (transform_output_iterator), what the algorithm computes in.
template <typename Out, typename Computed>
struct output_value {
  typedef typename std::conditional<std::is_void<typename iterator_value<Out>::type>::value, Computed,
                                    typename iterator_value<Out>::type>::type type;
};
}  // namespace detail

// The system an iterator belongs to: device_ptr -> device system, an iterator that names one
// (those built on thrust::iterator_facade do) -> that one, anything else -> host.
template <typename It, typename = void>
struct iterator_system { typedef thrust::host_system_tag type; };
template <typename It>
struct iterator_system<It, typename std::enable_if<!std::is_void<typename It::facade_system>::value>::type> {
  typedef typename It::facade_system type;
};
template <typename T>
struct iterator_system<device_ptr<T> > { typedef thrust::device_system_tag type; };

namespace detail {

template <typename It> struct is_device_iterator : std::false_type {};
template <typename T> struct is_device_iterator<device_ptr<T> > : std::true_type {};

// Iterators whose elements are computed (counting, constant, transform, permutation) derive from this.
struct fancy_iterator_marker {};
template <typename It>
struct is_fancy_iterator : std::is_base_of<fancy_iterator_marker, It> {};
// ... and those that take writes (discard_iterator) from this as well.
struct fancy_output_marker {};
template <typename It>
struct is_fancy_output_iterator : std::is_base_of<fancy_output_marker, It> {};

// An iterator type of the user's own, handed to kernels by value under a device policy: a
// class that is none of the library's iterators and that std::iterator_traits does not know
// (so not a container's iterator either).  Its operator[] and the assignment to what that
// returns must be callable in device code.
template <typename It, typename = void>
struct is_std_iterator : std::false_type {};
template <typename It>
struct is_std_iterator<It, typename std::enable_if<!std::is_void<typename std::iterator_traits<It>::iterator_category>::value>::type>
    : std::true_type {};
template <typename It>
struct is_user_device_iterator
    : std::integral_constant<bool, std::is_class<It>::value && std::is_trivially_copyable<It>::value &&
                                       !is_device_iterator<It>::value && !is_fancy_iterator<It>::value &&
                                       !is_std_iterator<It>::value> {};

// Raw address of the element an iterator points at.  Device iterators are device_ptr or,
// under an explicit device policy, plain pointers; host iterators must be contiguous
// (pointers, std::vector / host_vector iterators).
template <typename T> inline T* raw(const device_ptr<T>& p) { return p.get(); }
template <typename T> inline T* raw(T* p) { return p; }
template <typename It>
inline auto raw(It it) -> typename std::enable_if<
    !std::is_pointer<It>::value && !is_device_iterator<It>::value && !is_fancy_iterator<It>::value,
    typename std::remove_reference<decltype(*it)>::type*>::type {
  // never dereferences: callers pass begin() of a non-empty contiguous range or use n == 0
  return std::addressof(*it);
}
// (std::vector<bool> is bit-packed: its iterators point at no array of bool; a pure output
// iterator names no value type at all)
template <typename It, typename V>
struct is_vector_iterator_of
    : std::integral_constant<bool, std::is_same<It, typename std::vector<V>::iterator>::value ||
                                       std::is_same<It, typename std::vector<V>::const_iterator>::value> {};
template <typename It> struct is_vector_iterator_of<It, bool> : std::false_type {};
template <typename It> struct is_vector_iterator_of<It, void> : std::false_type {};
template <typename It>
struct is_contiguous_host_iterator
    : std::integral_constant<bool, std::is_pointer<It>::value ||
                                       is_vector_iterator_of<It, typename std::iterator_traits<It>::value_type>::value> {};
// raw(it) where the iterator has an address to give, a null pointer of the same type where it
// has none (for branches that are compiled for every iterator but only run for contiguous ones)
template <typename T, typename It>
inline T* raw_if(It it, std::true_type) { return const_cast<T*>(raw(it)); }
template <typename T, typename It>
inline T* raw_if(It, std::false_type) { return nullptr; }

template <typename T>
struct is_execution_policy : std::is_base_of<thrust::detail::execution_policy_marker,
                                             typename std::remove_cv<typename std::remove_reference<T>::type>::type> {};

// The policy a policy-less call uses for iterators of system tag Tag.
inline thrust::system::hip::tag& default_policy(thrust::device_system_tag) {
  static thrust::system::hip::tag t;
  return t;
}
inline thrust::system::cpp::tag& default_policy(thrust::host_system_tag) {
  static thrust::system::cpp::tag t;
  return t;
}
template <typename It>
inline auto policy_for() -> decltype(default_policy(typename iterator_system<It>::type())) {
  return default_policy(typename iterator_system<It>::type());
}

}  // namespace detail
}  // namespace thrust
