// thrust::iterator_facade: the operators of an iterator from a handful of members of the class
// that derives from it -- dereference(), equal(), increment(), decrement(), advance(n),
// distance_to(other) -- which may be private with thrust::iterator_core_access as a friend
// (thrust/iterator/iterator_facade.h:60-540).
//
// Every operator is __host__ __device__.  Under a device policy such an iterator is handed to
// kernels by value, as it is: what it holds must be usable in device code (device_ptr and
// device_vector iterators are, and so are the computed iterators of this library).
#pragma once
#include <cstddef>
#include <iterator>
#include <type_traits>

#include <thrust/detail/config.h>
#include <thrust/iterator/detail/fancy_iterator_base.h>
#include <thrust/iterator/iterator_categories.h>
#include <thrust/iterator/iterator_traits.h>

namespace thrust {

template <typename Derived, typename Value, typename System, typename Traversal, typename Reference,
          typename Difference = std::ptrdiff_t>
class iterator_facade;

// The one friend a derived iterator declares: the facade reaches the members through it.
class iterator_core_access {
  template <typename D, typename V, typename S, typename T, typename R, typename Df>
  friend class iterator_facade;

  template <typename F>
  __host__ __device__ static typename F::reference dereference(const F& f) { return f.dereference(); }
  template <typename F>
  __host__ __device__ static void increment(F& f) { f.increment(); }
  template <typename F>
  __host__ __device__ static void decrement(F& f) { f.decrement(); }
  template <typename F>
  __host__ __device__ static void advance(F& f, typename F::difference_type n) { f.advance(n); }
  template <typename F1, typename F2>
  __host__ __device__ static bool equal(const F1& a, const F2& b) { return a.equal(b); }
  // b - a
  template <typename F1, typename F2>
  __host__ __device__ static typename F1::difference_type distance_to(const F1& a, const F2& b) { return a.distance_to(b); }
};

template <typename Derived, typename Value, typename System, typename Traversal, typename Reference, typename Difference>
class iterator_facade : public detail::fancy_iterator_marker, public detail::fancy_output_marker {
 public:
  typedef typename std::remove_const<Value>::type value_type;
  typedef Reference reference;
  typedef void pointer;
  typedef Difference difference_type;
  typedef typename detail::category_of_traversal<Traversal>::type iterator_category;
  typedef System facade_system;  // what thrust::iterator_system answers for the derived iterator

  __host__ __device__ reference operator*() const { return iterator_core_access::dereference(self()); }
  __host__ __device__ reference operator[](difference_type n) const {
    Derived t(self());
    iterator_core_access::advance(t, n);
    return iterator_core_access::dereference(t);
  }
  __host__ __device__ Derived& operator++() { iterator_core_access::increment(self()); return self(); }
  __host__ __device__ Derived operator++(int) { Derived t(self()); iterator_core_access::increment(self()); return t; }
  __host__ __device__ Derived& operator--() { iterator_core_access::decrement(self()); return self(); }
  __host__ __device__ Derived operator--(int) { Derived t(self()); iterator_core_access::decrement(self()); return t; }
  __host__ __device__ Derived& operator+=(difference_type n) { iterator_core_access::advance(self(), n); return self(); }
  __host__ __device__ Derived& operator-=(difference_type n) { iterator_core_access::advance(self(), -n); return self(); }
  __host__ __device__ Derived operator+(difference_type n) const { Derived t(self()); iterator_core_access::advance(t, n); return t; }
  __host__ __device__ Derived operator-(difference_type n) const { Derived t(self()); iterator_core_access::advance(t, -n); return t; }
  __host__ __device__ friend Derived operator+(difference_type n, const Derived& it) { return it + n; }
  __host__ __device__ difference_type operator-(const Derived& o) const { return iterator_core_access::distance_to(o, self()); }
  __host__ __device__ bool operator==(const Derived& o) const { return iterator_core_access::equal(self(), o); }
  __host__ __device__ bool operator!=(const Derived& o) const { return !iterator_core_access::equal(self(), o); }
  __host__ __device__ bool operator<(const Derived& o) const { return iterator_core_access::distance_to(self(), o) > 0; }
  __host__ __device__ bool operator>(const Derived& o) const { return iterator_core_access::distance_to(self(), o) < 0; }
  __host__ __device__ bool operator<=(const Derived& o) const { return iterator_core_access::distance_to(self(), o) >= 0; }
  __host__ __device__ bool operator>=(const Derived& o) const { return iterator_core_access::distance_to(self(), o) <= 0; }

  // what a kernel receives: the iterator itself
  __host__ __device__ Derived device_view() const { return self(); }

 private:
  __host__ __device__ Derived& self() { return static_cast<Derived&>(*this); }
  __host__ __device__ const Derived& self() const { return static_cast<const Derived&>(*this); }
};

}  // namespace thrust
