// thrust::reverse_iterator: walks a range from its end towards its beginning; *it is the element
// before the wrapped position, as std::reverse_iterator (thrust/iterator/reverse_iterator.h,
// testing/reverse_iterator.cu).  It reads and writes what the wrapped iterator reads and writes
// and belongs to its system.
#pragma once
#include <thrust/iterator/detail/fancy_iterator_base.h>

namespace thrust {

template <typename It>
class reverse_iterator
    : public detail::fancy_iterator_base<reverse_iterator<It>, typename std::iterator_traits<It>::value_type,
                                         decltype(std::declval<const It&>()[std::ptrdiff_t(0)])> {
 public:
  typedef std::ptrdiff_t difference_type;
  typedef typename std::iterator_traits<It>::value_type value_type;
  typedef decltype(std::declval<const It&>()[std::ptrdiff_t(0)]) reference;
  typedef It iterator_type;
  __host__ __device__ reverse_iterator() : current_() {}
  __host__ __device__ explicit reverse_iterator(It position) : current_(position) {}
  template <typename Other>
  __host__ __device__ reverse_iterator(const reverse_iterator<Other>& other) : current_(other.base()) {}
  __host__ __device__ It base() const { return current_; }
  __host__ __device__ reference at(difference_type i) const { return current_[-1 - i]; }
  __host__ __device__ void advance(difference_type n) { current_ -= n; }
  __host__ __device__ difference_type distance_to(const reverse_iterator& o) const { return current_ - o.current_; }
  // a template so that it only exists for iterators that have a device view
  template <typename I = It>
  reverse_iterator<typename detail::device_view_of<I>::type> device_view() const {
    return reverse_iterator<typename detail::device_view_of<I>::type>(detail::device_view(current_));
  }

 private:
  It current_;
};
template <typename It>
inline reverse_iterator<It> make_reverse_iterator(It position) {
  return reverse_iterator<It>(position);
}

template <typename It>
struct iterator_system<reverse_iterator<It> > {
  typedef typename iterator_system<It>::type type;
};

}  // namespace thrust
