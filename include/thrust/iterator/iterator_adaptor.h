// thrust::iterator_adaptor: an iterator that behaves like the one it wraps except for the members
// the deriving class writes anew -- usually dereference(), sometimes advance() and distance_to()
// (thrust/iterator/iterator_adaptor.h:40-240; the repeat_iterator of its documentation is the
// model of a use).  Value, System, Traversal, Reference and Difference default to the wrapped
// iterator's.
#pragma once
#include <thrust/iterator/iterator_facade.h>

namespace thrust {
namespace detail {
template <typename Given, typename Else>
struct given_or { typedef Given type; };
template <typename Else>
struct given_or<use_default, Else> { typedef Else type; };

template <typename Base, typename Value, typename Reference>
struct adaptor_reference {  // the caller's, else Value& if a value type is named, else the wrapped iterator's
  typedef typename given_or<Reference,
                            typename std::conditional<std::is_same<Value, use_default>::value,
                                                      decltype(*std::declval<const Base&>()),
                                                      typename given_or<Value, int>::type&>::type>::type type;
};
template <typename Base, typename Traversal>
struct adaptor_traversal {
  typedef typename given_or<Traversal, typename std::iterator_traits<Base>::iterator_category>::type type;
};
}  // namespace detail

template <typename Derived, typename Base, typename Value = use_default, typename System = use_default,
          typename Traversal = use_default, typename Reference = use_default, typename Difference = use_default>
class iterator_adaptor
    : public iterator_facade<Derived, typename detail::given_or<Value, typename thrust::iterator_value<Base>::type>::type,
                             typename detail::given_or<System, typename thrust::iterator_system<Base>::type>::type,
                             typename detail::adaptor_traversal<Base, Traversal>::type,
                             typename detail::adaptor_reference<Base, Value, Reference>::type,
                             typename detail::given_or<Difference, typename thrust::iterator_difference<Base>::type>::type> {
  friend class thrust::iterator_core_access;

 public:
  typedef Base base_type;
  typedef typename detail::adaptor_reference<Base, Value, Reference>::type reference;
  typedef typename detail::given_or<Difference, typename thrust::iterator_difference<Base>::type>::type difference_type;

  __host__ __device__ iterator_adaptor() : m_iterator() {}
  __host__ __device__ explicit iterator_adaptor(const Base& it) : m_iterator(it) {}
  __host__ __device__ const Base& base() const { return m_iterator; }

 protected:
  typedef iterator_adaptor super_t;  // what deriving classes call their base
  __host__ __device__ const Base& base_reference() const { return m_iterator; }
  __host__ __device__ Base& base_reference() { return m_iterator; }

 private:
  // the members the facade asks for, as the wrapped iterator answers them
  __host__ __device__ reference dereference() const { return *m_iterator; }
  template <typename Other>
  __host__ __device__ bool equal(const Other& o) const { return m_iterator == o.base(); }
  __host__ __device__ void advance(difference_type n) { m_iterator += n; }
  __host__ __device__ void increment() { ++m_iterator; }
  __host__ __device__ void decrement() { --m_iterator; }
  template <typename Other>
  __host__ __device__ difference_type distance_to(const Other& o) const { return o.base() - m_iterator; }

  Base m_iterator;
};

}  // namespace thrust
