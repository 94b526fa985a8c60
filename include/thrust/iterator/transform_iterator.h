// thrust::transform_iterator: element i is f(base[i]) (thrust/iterator/transform_iterator.h).
// It belongs to the system of the iterator it wraps.
#pragma once
#include <thrust/iterator/detail/fancy_iterator_base.h>

namespace thrust {

namespace detail {
// The element type: the caller's Value if one is named, else the caller's Reference without its
// qualifiers, else whatever F returns for an element of It
// (thrust/iterator/detail/transform_iterator.inl:27-60).
template <typename F, typename It, typename Reference = use_default, typename Value = use_default>
struct transform_result {
  typedef typename std::decay<Value>::type type;
};
template <typename F, typename It, typename Reference>
struct transform_result<F, It, Reference, use_default> {
  typedef typename std::decay<Reference>::type type;
};
template <typename F, typename It>
struct transform_result<F, It, use_default, use_default> {
  typedef typename std::decay<decltype(std::declval<F&>()(
      std::declval<typename std::iterator_traits<It>::value_type>()))>::type type;
};
}  // namespace detail

template <typename F, typename It, typename Reference = use_default, typename Value = use_default>
class transform_iterator
    : public detail::fancy_iterator_base<transform_iterator<F, It, Reference, Value>,
                                         typename detail::transform_result<F, It, Reference, Value>::type> {
 public:
  typedef std::ptrdiff_t difference_type;
  typedef typename detail::transform_result<F, It, Reference, Value>::type value_type;
  __host__ __device__ transform_iterator() : it_(), f_() {}
  __host__ __device__ transform_iterator(It it, F f) : it_(it), f_(f) {}
  __host__ __device__ value_type at(difference_type i) const {
    return f_(static_cast<typename std::iterator_traits<It>::value_type>(it_[i]));
  }
  __host__ __device__ void advance(difference_type n) { it_ += n; }
  __host__ __device__ difference_type distance_to(const transform_iterator& o) const { return o.it_ - it_; }
  __host__ __device__ It base() const { return it_; }
  // a template so that it only exists for iterators that have a device view
  template <typename I = It>
  transform_iterator<F, typename detail::device_view_of<I>::type, Reference, Value> device_view() const {
    return transform_iterator<F, typename detail::device_view_of<I>::type, Reference, Value>(detail::device_view(it_), f_);
  }

 private:
  It it_;
  mutable F f_;
};
template <typename F, typename It>
inline transform_iterator<F, It> make_transform_iterator(It it, F f) { return transform_iterator<F, It>(it, f); }

template <typename F, typename It, typename R, typename V>
struct iterator_system<transform_iterator<F, It, R, V> > { typedef typename iterator_system<It>::type type; };

}  // namespace thrust
