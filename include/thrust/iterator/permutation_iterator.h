// thrust::permutation_iterator: element i is elements[indices[i]]
// (thrust/iterator/permutation_iterator.h); the read side of gather and, over an array, a
// range that can be written and sorted through (dereferencing yields what the element
// iterator yields: a reference for arrays).  It belongs to the system of the element iterator.
#pragma once
#include <thrust/iterator/detail/fancy_iterator_base.h>

namespace thrust {

template <typename ElementIt, typename IndexIt>
class permutation_iterator
    : public detail::fancy_iterator_base<permutation_iterator<ElementIt, IndexIt>,
                                         typename std::iterator_traits<ElementIt>::value_type,
                                         decltype(std::declval<const ElementIt&>()[std::ptrdiff_t(0)])> {
 public:
  typedef std::ptrdiff_t difference_type;
  typedef typename std::iterator_traits<ElementIt>::value_type value_type;
  typedef decltype(std::declval<const ElementIt&>()[std::ptrdiff_t(0)]) reference;
  __host__ __device__ permutation_iterator() : elements_(), indices_() {}
  __host__ __device__ permutation_iterator(ElementIt elements, IndexIt indices) : elements_(elements), indices_(indices) {}
  __host__ __device__ reference at(difference_type i) const {
    return elements_[(difference_type) static_cast<typename std::iterator_traits<IndexIt>::value_type>(indices_[i])];
  }
  __host__ __device__ void advance(difference_type n) { indices_ += n; }
  __host__ __device__ difference_type distance_to(const permutation_iterator& o) const { return o.indices_ - indices_; }
  // a template so that it only exists for iterators that have a device view
  template <typename E = ElementIt, typename I = IndexIt>
  permutation_iterator<typename detail::device_view_of<E>::type, typename detail::device_view_of<I>::type>
  device_view() const {
    return permutation_iterator<typename detail::device_view_of<E>::type, typename detail::device_view_of<I>::type>(
        detail::device_view(elements_), detail::device_view(indices_));
  }

 private:
  ElementIt elements_;
  IndexIt indices_;
};
template <typename ElementIt, typename IndexIt>
inline permutation_iterator<ElementIt, IndexIt> make_permutation_iterator(ElementIt e, IndexIt i) {
  return permutation_iterator<ElementIt, IndexIt>(e, i);
}

template <typename ElementIt, typename IndexIt>
struct iterator_system<permutation_iterator<ElementIt, IndexIt> > {
  typedef typename iterator_system<ElementIt>::type type;
};

}  // namespace thrust
