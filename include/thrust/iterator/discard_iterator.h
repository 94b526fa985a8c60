// thrust::discard_iterator: an output that throws away whatever is assigned through it, for
// the half of an algorithm's result a caller does not want (thrust/iterator/discard_iterator.h).
// Reading it yields a default-constructed value.
#pragma once
#include <thrust/iterator/detail/fancy_iterator_base.h>

namespace thrust {

namespace detail {
// what dereferencing a discard_iterator gives: assignable from anything, convertible to the value
template <typename T>
struct discard_reference {
  template <typename V>
  __host__ __device__ const discard_reference& operator=(const V&) const { return *this; }
  __host__ __device__ operator T() const { return T(); }
};
}  // namespace detail

template <typename T = int>
class discard_iterator : public detail::fancy_iterator_base<discard_iterator<T>, T, detail::discard_reference<T> >,
                         public detail::fancy_output_marker {
 public:
  typedef std::ptrdiff_t difference_type;
  __host__ __device__ discard_iterator() : index_(0) {}
  __host__ __device__ explicit discard_iterator(difference_type index) : index_(index) {}
  __host__ __device__ detail::discard_reference<T> at(difference_type) const { return detail::discard_reference<T>(); }
  __host__ __device__ void advance(difference_type n) { index_ += n; }
  __host__ __device__ difference_type distance_to(const discard_iterator& o) const { return o.index_ - index_; }
  __host__ __device__ discard_iterator device_view() const { return *this; }

 private:
  difference_type index_;
};
__host__ __device__ inline discard_iterator<> make_discard_iterator(std::ptrdiff_t index = 0) {
  return discard_iterator<>(index);
}

template <typename T>
struct iterator_system<discard_iterator<T> > { typedef thrust::device_system_tag type; };

}  // namespace thrust
