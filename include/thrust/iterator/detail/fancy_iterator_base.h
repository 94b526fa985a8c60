// Common part of the fancy iterators (counting, constant, transform, permutation): a
// random-access iterator whose element i is computed, not stored
// (thrust/iterator/iterator_facade.h and iterator_adaptor.h in the reference).
//
// Every member is __host__ __device__: the same object is walked by the sequential host
// system and passed by value into the device system's kernels, which exist in translation
// units compiled with hipcc (thrust/system/hip/detail/fancy_kernels.h).
#pragma once
#include <cstddef>
#include <iterator>
#include <type_traits>
#include <utility>

#include <thrust/detail/config.h>
#include <thrust/iterator/iterator_traits.h>

namespace thrust {
// "Work it out from the other arguments" (thrust/iterator/iterator_adaptor.h of the reference).
struct use_default {};

namespace detail {

// Derived provides: Reference at(difference_type i) const  (element i from the current position)
//                   void advance(difference_type n)
//                   difference_type distance_to(const Derived& other) const  (other - *this)
template <typename Derived, typename Value, typename Reference = Value>
class fancy_iterator_base : public fancy_iterator_marker {
 public:
  typedef std::random_access_iterator_tag iterator_category;
  typedef Value value_type;
  typedef std::ptrdiff_t difference_type;
  typedef void pointer;
  typedef Reference reference;

  __host__ __device__ Reference operator*() const { return self().at(0); }
  __host__ __device__ Reference operator[](difference_type i) const { return self().at(i); }
  __host__ __device__ Derived& operator++() { self().advance(1); return self(); }
  __host__ __device__ Derived operator++(int) { Derived t(self()); self().advance(1); return t; }
  __host__ __device__ Derived& operator--() { self().advance(-1); return self(); }
  __host__ __device__ Derived operator--(int) { Derived t(self()); self().advance(-1); return t; }
  __host__ __device__ Derived& operator+=(difference_type n) { self().advance(n); return self(); }
  __host__ __device__ Derived& operator-=(difference_type n) { self().advance(-n); return self(); }
  __host__ __device__ Derived operator+(difference_type n) const { Derived t(self()); t.advance(n); return t; }
  __host__ __device__ Derived operator-(difference_type n) const { Derived t(self()); t.advance(-n); return t; }
  __host__ __device__ difference_type operator-(const Derived& o) const { return o.distance_to(self()); }
  __host__ __device__ bool operator==(const Derived& o) const { return self().distance_to(o) == 0; }
  __host__ __device__ bool operator!=(const Derived& o) const { return self().distance_to(o) != 0; }
  __host__ __device__ bool operator<(const Derived& o) const { return self().distance_to(o) > 0; }
  __host__ __device__ bool operator>(const Derived& o) const { return self().distance_to(o) < 0; }
  __host__ __device__ bool operator<=(const Derived& o) const { return self().distance_to(o) >= 0; }
  __host__ __device__ bool operator>=(const Derived& o) const { return self().distance_to(o) <= 0; }

 private:
  __host__ __device__ Derived& self() { return static_cast<Derived&>(*this); }
  __host__ __device__ const Derived& self() const { return static_cast<const Derived&>(*this); }
};

// What a kernel receives for an iterator: device_ptr becomes the raw pointer (its
// dereference is a host-side proxy), fancy iterators convert the iterators they wrap.
template <typename T> inline T* device_view(T* p) { return p; }
template <typename T> inline T* device_view(const device_ptr<T>& p) { return p.get(); }
template <typename It>
inline auto device_view(const It& it) -> decltype(it.device_view()) { return it.device_view(); }
// an iterator type of the user's own travels as it is
template <typename It>
inline typename std::enable_if<is_user_device_iterator<It>::value, It>::type device_view(const It& it) { return it; }
template <typename It>
struct device_view_of { typedef decltype(device_view(std::declval<const It&>())) type; };

}  // namespace detail
}  // namespace thrust
