// thrust::counting_iterator: element i is start + i (thrust/iterator/counting_iterator.h).
// It belongs to the device system when no policy says otherwise, as "any system" does in
// the reference.
#pragma once
#include <thrust/iterator/detail/fancy_iterator_base.h>

namespace thrust {

// System: the system the range belongs to when no policy says so (host_system_tag for the
// sequential loops); Traversal and Difference are accepted for source compatibility
// (thrust/iterator/counting_iterator.h:135-139).
template <typename T, typename System = use_default, typename Traversal = use_default, typename Difference = use_default>
class counting_iterator : public detail::fancy_iterator_base<counting_iterator<T, System, Traversal, Difference>, T> {
 public:
  typedef std::ptrdiff_t difference_type;
  __host__ __device__ counting_iterator() : value_() {}
  __host__ __device__ explicit counting_iterator(T v) : value_(v) {}
  __host__ __device__ T at(difference_type i) const { return (T)(value_ + (T)i); }
  __host__ __device__ void advance(difference_type n) { value_ = (T)(value_ + (T)n); }
  __host__ __device__ difference_type distance_to(const counting_iterator& o) const {
    return (difference_type)o.value_ - (difference_type)value_;
  }
  __host__ __device__ counting_iterator device_view() const { return *this; }

 private:
  T value_;
};
template <typename T>
__host__ __device__ inline counting_iterator<T> make_counting_iterator(T v) { return counting_iterator<T>(v); }

template <typename T, typename S, typename Tr, typename D>
struct iterator_system<counting_iterator<T, S, Tr, D> > {
  typedef typename std::conditional<std::is_same<S, use_default>::value, thrust::device_system_tag, S>::type type;
};

}  // namespace thrust
