// thrust::transform_output_iterator: an output iterator that applies a function to what is assigned
// through it and hands the result to the iterator it wraps
// (thrust/iterator/transform_output_iterator.h, detail/transform_output_iterator.inl;
// testing/transform_output_iterator.cu).
#pragma once
#include <thrust/iterator/detail/fancy_iterator_base.h>

namespace thrust {
namespace detail {
// what dereferencing yields: assignment transforms and forwards
template <typename F, typename Out>
class transform_output_proxy {
 public:
  __host__ __device__ transform_output_proxy(const Out& out, F f) : out_(out), f_(f) {}
  template <typename T>
  __host__ __device__ const transform_output_proxy& operator=(const T& x) const {
    *out_ = f_(x);
    return *this;
  }

 private:
  Out out_;
  mutable F f_;
};
}  // namespace detail

template <typename F, typename Out>
class transform_output_iterator
    : public detail::fancy_iterator_base<transform_output_iterator<F, Out>, void, detail::transform_output_proxy<F, Out> >,
      public detail::fancy_output_marker {
 public:
  typedef std::ptrdiff_t difference_type;
  typedef detail::transform_output_proxy<F, Out> reference;
  __host__ __device__ transform_output_iterator() : out_(), f_() {}
  __host__ __device__ transform_output_iterator(const Out& out, F f) : out_(out), f_(f) {}
  __host__ __device__ reference at(difference_type i) const { return reference(out_ + i, f_); }
  __host__ __device__ void advance(difference_type n) { out_ += n; }
  __host__ __device__ difference_type distance_to(const transform_output_iterator& o) const { return o.out_ - out_; }
  __host__ __device__ const Out& base() const { return out_; }
  // a template so that it only exists for iterators that have a device view
  template <typename O = Out>
  transform_output_iterator<F, typename detail::device_view_of<O>::type> device_view() const {
    return transform_output_iterator<F, typename detail::device_view_of<O>::type>(detail::device_view(out_), f_);
  }

 private:
  Out out_;
  mutable F f_;
};
template <typename F, typename Out>
inline transform_output_iterator<F, Out> make_transform_output_iterator(Out out, F f) {
  return transform_output_iterator<F, Out>(out, f);
}

template <typename F, typename Out>
struct iterator_system<transform_output_iterator<F, Out> > {
  typedef typename iterator_system<Out>::type type;
};

}  // namespace thrust
