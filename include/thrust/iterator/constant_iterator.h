// thrust::constant_iterator: every element is the same value
// (thrust/iterator/constant_iterator.h).
#pragma once
#include <thrust/iterator/detail/fancy_iterator_base.h>

namespace thrust {

template <typename T>
class constant_iterator : public detail::fancy_iterator_base<constant_iterator<T>, T> {
 public:
  typedef std::ptrdiff_t difference_type;
  __host__ __device__ constant_iterator() : value_(), index_(0) {}
  __host__ __device__ explicit constant_iterator(T v, difference_type index = 0) : value_(v), index_(index) {}
  __host__ __device__ T at(difference_type) const { return value_; }
  __host__ __device__ void advance(difference_type n) { index_ += n; }
  __host__ __device__ difference_type distance_to(const constant_iterator& o) const { return o.index_ - index_; }
  __host__ __device__ constant_iterator device_view() const { return *this; }

 private:
  T value_;
  difference_type index_;
};
template <typename T>
__host__ __device__ inline constant_iterator<T> make_constant_iterator(T v) { return constant_iterator<T>(v); }

template <typename T>
struct iterator_system<constant_iterator<T> > { typedef thrust::device_system_tag type; };

}  // namespace thrust
