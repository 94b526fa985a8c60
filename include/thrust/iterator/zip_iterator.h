// thrust::zip_iterator: element i is the tuple (it0[i], it1[i], ...)
// (thrust/iterator/zip_iterator.h).  Dereferencing yields a tuple of references, so a
// kernel can write through it; its value type is the tuple of the value types.  It belongs
// to the system of its first iterator.
#pragma once
#include <thrust/iterator/detail/fancy_iterator_base.h>
#include <thrust/tuple.h>

namespace thrust {

template <typename IteratorTuple>
class zip_iterator;

namespace detail {
template <typename It>
struct zip_reference_of { typedef decltype(*std::declval<const It&>()) type; };

template <typename Tuple>
struct zip_traits;
template <typename... Its>
struct zip_traits<tuple<Its...> > {
  typedef tuple<typename std::iterator_traits<Its>::value_type...> value_type;
  typedef tuple<typename zip_reference_of<Its>::type...> reference;
};
// only for iterators that have a device view (host iterators do not)
template <typename Tuple>
struct zip_view_tuple;
template <typename... Its>
struct zip_view_tuple<tuple<Its...> > { typedef tuple<typename device_view_of<Its>::type...> type; };

// element-wise helpers over the iterator tuple
__host__ __device__ inline void zip_advance(tuple<>&, std::ptrdiff_t) {}
template <typename H, typename... T>
__host__ __device__ inline void zip_advance(tuple<H, T...>& its, std::ptrdiff_t n) {
  its.head += n;
  zip_advance(its.tail, n);
}
__host__ __device__ inline tuple<> zip_deref(const tuple<>&, std::ptrdiff_t) { return tuple<>(); }
template <typename H, typename... T>
__host__ __device__ inline tuple<typename zip_reference_of<H>::type, typename zip_reference_of<T>::type...> zip_deref(
    const tuple<H, T...>& its, std::ptrdiff_t i) {
  typedef tuple<typename zip_reference_of<H>::type, typename zip_reference_of<T>::type...> R;
  return R(typename R::cons_tag(), its.head[i], zip_deref(its.tail, i));
}
inline tuple<> zip_views(const tuple<>&) { return tuple<>(); }
template <typename H, typename... T>
inline tuple<typename device_view_of<H>::type, typename device_view_of<T>::type...> zip_views(const tuple<H, T...>& its) {
  typedef tuple<typename device_view_of<H>::type, typename device_view_of<T>::type...> R;
  return R(typename R::cons_tag(), device_view(its.head), zip_views(its.tail));
}
}  // namespace detail

template <typename IteratorTuple>
class zip_iterator : public detail::fancy_iterator_base<zip_iterator<IteratorTuple>,
                                                        typename detail::zip_traits<IteratorTuple>::value_type,
                                                        typename detail::zip_traits<IteratorTuple>::reference> {
 public:
  typedef std::ptrdiff_t difference_type;
  typedef typename detail::zip_traits<IteratorTuple>::reference reference;
  __host__ __device__ zip_iterator() {}
  __host__ __device__ explicit zip_iterator(const IteratorTuple& its) : its_(its) {}
  __host__ __device__ reference at(difference_type i) const { return detail::zip_deref(its_, i); }
  __host__ __device__ void advance(difference_type n) { detail::zip_advance(its_, n); }
  __host__ __device__ difference_type distance_to(const zip_iterator& o) const { return o.its_.head - its_.head; }
  __host__ __device__ const IteratorTuple& get_iterator_tuple() const { return its_; }
  // a template so that it only exists for iterators that have a device view
  template <typename Its = IteratorTuple>
  zip_iterator<typename detail::zip_view_tuple<Its>::type> device_view() const {
    return zip_iterator<typename detail::zip_view_tuple<Its>::type>(detail::zip_views(its_));
  }

 private:
  IteratorTuple its_;
};

template <typename... Its>
inline zip_iterator<tuple<Its...> > make_zip_iterator(const tuple<Its...>& its) {
  return zip_iterator<tuple<Its...> >(its);
}
template <typename... Its>
inline zip_iterator<tuple<Its...> > make_zip_iterator(Its... its) {
  return zip_iterator<tuple<Its...> >(tuple<Its...>(its...));
}

template <typename H, typename... T>
struct iterator_system<zip_iterator<tuple<H, T...> > > { typedef typename iterator_system<H>::type type; };

}  // namespace thrust
