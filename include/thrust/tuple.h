// thrust::tuple, thrust::get, thrust::make_tuple, thrust::tie, tuple_size, tuple_element.
//
// A small tuple whose every member is __host__ __device__ (thrust/tuple.h in the
// reference): it is the value type and the reference type of zip_iterator, so it must be
// constructible, assignable and comparable inside kernels.  Elements may be references
// (what dereferencing a zip_iterator yields); assigning to such a tuple writes through them.
#pragma once
#include <cstddef>
#include <type_traits>
#include <utility>

#include <thrust/detail/config.h>

namespace thrust {

template <typename... Ts>
class tuple;

template <>
class tuple<> {
 public:
  __host__ __device__ tuple() {}
  tuple(const tuple&) = default;
  __host__ __device__ const tuple& operator=(const tuple&) const { return *this; }
  __host__ __device__ bool equal(const tuple&) const { return true; }
  __host__ __device__ bool less(const tuple&) const { return false; }
};

template <typename H, typename... T>
class tuple<H, T...> {
 public:
  H head;
  // the empty tuple that ends every chain takes no room: tuple<float, float> is 8 bytes
  [[no_unique_address]] tuple<T...> tail;

  struct cons_tag {};
  __host__ __device__ tuple() : head(), tail() {}
  // (defaulted: a tuple of plain values is copied as its bytes are, also by device code that
  // moves elements without knowing their type)
  tuple(const tuple& o) = default;
  // from the first element and the tuple of the others
  template <typename HH>
  __host__ __device__ tuple(cons_tag, HH&& h, const tuple<T...>& t) : head(static_cast<HH&&>(h)), tail(t) {}
  template <typename H2, typename... T2,
            typename = typename std::enable_if<sizeof...(T2) == sizeof...(T) && std::is_convertible<H2, H>::value>::type>
  __host__ __device__ tuple(H2&& h, T2&&... t) : head(static_cast<H2&&>(h)), tail(static_cast<T2&&>(t)...) {}
  // from a tuple of other element types (values from references and the other way round)
  template <typename H2, typename... T2, typename = typename std::enable_if<sizeof...(T2) == sizeof...(T)>::type>
  __host__ __device__ tuple(const tuple<H2, T2...>& o) : head(o.head), tail(o.tail) {}
  template <typename H2, typename... T2, typename = typename std::enable_if<sizeof...(T2) == sizeof...(T)>::type>
  __host__ __device__ tuple(tuple<H2, T2...>& o) : head(o.head), tail(o.tail) {}

  __host__ __device__ tuple& operator=(const tuple& o) {
    head = o.head;
    tail = o.tail;
    return *this;
  }
  template <typename H2, typename... T2>
  __host__ __device__ tuple& operator=(const tuple<H2, T2...>& o) {
    head = o.head;
    tail = o.tail;
    return *this;
  }
  // a tuple of references is assigned through even when it is a temporary or const
  template <typename H2, typename... T2>
  __host__ __device__ const tuple& operator=(const tuple<H2, T2...>& o) const {
    head = o.head;
    tail = o.tail;
    return *this;
  }

  template <typename H2, typename... T2>
  __host__ __device__ bool equal(const tuple<H2, T2...>& o) const { return head == o.head && tail.equal(o.tail); }
  template <typename H2, typename... T2>
  __host__ __device__ bool less(const tuple<H2, T2...>& o) const {
    if (head < o.head) return true;
    if (o.head < head) return false;
    return tail.less(o.tail);
  }
};

template <typename... A, typename... B>
__host__ __device__ inline bool operator==(const tuple<A...>& a, const tuple<B...>& b) { return a.equal(b); }
template <typename... A, typename... B>
__host__ __device__ inline bool operator!=(const tuple<A...>& a, const tuple<B...>& b) { return !a.equal(b); }
template <typename... A, typename... B>
__host__ __device__ inline bool operator<(const tuple<A...>& a, const tuple<B...>& b) { return a.less(b); }
template <typename... A, typename... B>
__host__ __device__ inline bool operator>(const tuple<A...>& a, const tuple<B...>& b) { return b.less(a); }
template <typename... A, typename... B>
__host__ __device__ inline bool operator<=(const tuple<A...>& a, const tuple<B...>& b) { return !b.less(a); }
template <typename... A, typename... B>
__host__ __device__ inline bool operator>=(const tuple<A...>& a, const tuple<B...>& b) { return !a.less(b); }

template <typename Tuple>
struct tuple_size;
template <typename... Ts>
struct tuple_size<tuple<Ts...> > : std::integral_constant<std::size_t, sizeof...(Ts)> {};
template <typename Tuple>
struct tuple_size<const Tuple> : tuple_size<Tuple> {};

template <std::size_t I, typename Tuple>
struct tuple_element;
template <typename H, typename... T>
struct tuple_element<0, tuple<H, T...> > { typedef H type; };
template <std::size_t I, typename H, typename... T>
struct tuple_element<I, tuple<H, T...> > : tuple_element<I - 1, tuple<T...> > {};
template <std::size_t I, typename Tuple>
struct tuple_element<I, const Tuple> : tuple_element<I, Tuple> {};

namespace detail {
template <std::size_t I>
struct tuple_get {
  template <typename H, typename... T>
  __host__ __device__ static typename tuple_element<I, tuple<H, T...> >::type& at(tuple<H, T...>& t) {
    return tuple_get<I - 1>::at(t.tail);
  }
  template <typename H, typename... T>
  __host__ __device__ static const typename tuple_element<I, tuple<H, T...> >::type& at(const tuple<H, T...>& t) {
    return tuple_get<I - 1>::at(t.tail);
  }
};
template <>
struct tuple_get<0> {
  template <typename H, typename... T>
  __host__ __device__ static H& at(tuple<H, T...>& t) { return t.head; }
  template <typename H, typename... T>
  __host__ __device__ static const H& at(const tuple<H, T...>& t) { return t.head; }
};
}  // namespace detail

// get<I> of a tuple of references yields the referenced object, also through a const tuple
template <std::size_t I, typename... Ts>
__host__ __device__ inline typename tuple_element<I, tuple<Ts...> >::type& get(tuple<Ts...>& t) {
  return detail::tuple_get<I>::at(t);
}
template <std::size_t I, typename... Ts>
__host__ __device__ inline
    typename std::conditional<std::is_reference<typename tuple_element<I, tuple<Ts...> >::type>::value,
                              typename tuple_element<I, tuple<Ts...> >::type,
                              const typename tuple_element<I, tuple<Ts...> >::type&>::type
    get(const tuple<Ts...>& t) {
  return detail::tuple_get<I>::at(t);
}

template <typename... Ts>
__host__ __device__ inline tuple<typename std::decay<Ts>::type...> make_tuple(Ts&&... v) {
  return tuple<typename std::decay<Ts>::type...>(static_cast<Ts&&>(v)...);
}
template <typename... Ts>
__host__ __device__ inline tuple<Ts&...> tie(Ts&... v) {
  return tuple<Ts&...>(v...);
}

}  // namespace thrust
