// thrust::transform_input_output_iterator: reads give input_function(element), writes store
// output_function(value) (thrust/iterator/transform_input_output_iterator.h,
// detail/transform_input_output_iterator.inl; testing/transform_input_output_iterator.cu).
#pragma once
#include <thrust/iterator/detail/fancy_iterator_base.h>

namespace thrust {
namespace detail {
// what dereferencing yields: converts to the transformed element, assignment transforms back
template <typename In, typename OutF, typename It>
class transform_input_output_proxy {
 public:
  typedef typename std::decay<decltype(std::declval<In&>()(
      std::declval<typename std::iterator_traits<It>::value_type>()))>::type value_type;
  __host__ __device__ transform_input_output_proxy(const It& it, In in, OutF out) : it_(it), in_(in), out_(out) {}
  __host__ __device__ operator value_type() const {
    return in_(static_cast<typename std::iterator_traits<It>::value_type>(*it_));
  }
  template <typename T>
  __host__ __device__ const transform_input_output_proxy& operator=(const T& x) const {
    *it_ = out_(x);
    return *this;
  }
  __host__ __device__ const transform_input_output_proxy& operator=(const transform_input_output_proxy& x) const {
    *it_ = *x.it_;
    return *this;
  }

 private:
  It it_;
  mutable In in_;
  mutable OutF out_;
};
}  // namespace detail

template <typename In, typename OutF, typename It>
class transform_input_output_iterator
    : public detail::fancy_iterator_base<transform_input_output_iterator<In, OutF, It>,
                                         typename detail::transform_input_output_proxy<In, OutF, It>::value_type,
                                         detail::transform_input_output_proxy<In, OutF, It> >,
      public detail::fancy_output_marker {
 public:
  typedef std::ptrdiff_t difference_type;
  typedef detail::transform_input_output_proxy<In, OutF, It> reference;
  __host__ __device__ transform_input_output_iterator() : it_(), in_(), out_() {}
  __host__ __device__ transform_input_output_iterator(const It& it, In in, OutF out) : it_(it), in_(in), out_(out) {}
  __host__ __device__ reference at(difference_type i) const { return reference(it_ + i, in_, out_); }
  __host__ __device__ void advance(difference_type n) { it_ += n; }
  __host__ __device__ difference_type distance_to(const transform_input_output_iterator& o) const { return o.it_ - it_; }
  __host__ __device__ const It& base() const { return it_; }
  // a template so that it only exists for iterators that have a device view
  template <typename I = It>
  transform_input_output_iterator<In, OutF, typename detail::device_view_of<I>::type> device_view() const {
    return transform_input_output_iterator<In, OutF, typename detail::device_view_of<I>::type>(detail::device_view(it_),
                                                                                               in_, out_);
  }

 private:
  It it_;
  mutable In in_;
  mutable OutF out_;
};
template <typename In, typename OutF, typename It>
inline transform_input_output_iterator<In, OutF, It> make_transform_input_output_iterator(It it, In in, OutF out) {
  return transform_input_output_iterator<In, OutF, It>(it, in, out);
}
template <typename In, typename OutF, typename It>
struct iterator_system<transform_input_output_iterator<In, OutF, It> > {
  typedef typename iterator_system<It>::type type;
};
}  // namespace thrust
