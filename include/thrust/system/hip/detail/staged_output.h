// Outputs of the by-key algorithms (reduce_by_key, unique_copy, unique_by_key_copy) that are not
// arrays in device memory: a discard_iterator for the half of the result nobody wants, a zip
// of arrays, a caller's own iterator type.  The reference's agents write through the iterator
// itself (thrust/system/cuda/detail/reduce_by_key.h:520-600, unique_by_key.h:380-470); here
// the algorithm writes an array in temporary storage and one copy carries the result through
// the iterator afterwards (nothing is copied into a discard_iterator).  An array in device
// memory is used where it lies.
#pragma once
#include <thrust/device_ptr.h>
#include <thrust/iterator/discard_iterator.h>
#include <thrust/system/hip/detail/backend.h>

namespace thrust {

template <typename D, typename In, typename Out>
Out copy(const detail::execution_policy_base<D>& exec, In first, In last, Out result);

namespace system {
namespace hip {
namespace detail {

template <typename It>
struct is_memory_iterator
    : std::integral_constant<bool, std::is_pointer<It>::value || thrust::detail::is_device_iterator<It>::value> {};
template <typename T, typename Out>
struct is_array_of : std::integral_constant<bool, is_memory_iterator<Out>::value &&
                                                      std::is_same<typename iterator_value<Out>::type, T>::value> {};

template <typename It> struct is_discard_iterator : std::false_type {};
template <typename T> struct is_discard_iterator<thrust::discard_iterator<T> > : std::true_type {};

// The element type to compute for output Out when the algorithm's own result type is V: a
// discard_iterator takes anything, every other output names its type.
template <typename Out, typename V>
struct staged_value { typedef typename iterator_value<Out>::type type; };
template <typename T, typename V>
struct staged_value<thrust::discard_iterator<T>, V> { typedef V type; };

template <typename Out, typename V, bool Memory = is_memory_iterator<Out>::value>
class output_stage {
 public:
  typedef Out iterator;
  output_stage(void*, const temp_source&, Out out, uint64_t) : out_(out) {}
  Out begin() const { return out_; }
  template <typename Exec>
  Out finish(Exec&, uint64_t count) const { return out_ + count; }

 private:
  Out out_;
};
template <typename Out, typename V>
class output_stage<Out, V, false> {
  typedef typename staged_value<Out, V>::type E;

 public:
  typedef thrust::device_ptr<E> iterator;
  // capacity: the most elements the algorithm may write
  output_stage(void* stream, const temp_source& source, Out out, uint64_t capacity) : holder_(stream, source), out_(out) {
    holder_.ensure((std::size_t)(capacity ? capacity : 1) * sizeof(E));
  }
  iterator begin() const { return iterator(static_cast<E*>(holder_.ptr())); }
  template <typename Exec>
  Out finish(Exec& exec, uint64_t count) const {
    if (!is_discard_iterator<Out>::value && count) thrust::copy(exec, begin(), begin() + count, out_);
    return out_ + count;
  }

 private:
  temp_storage holder_;
  Out out_;
};

}  // namespace detail
}  // namespace hip
}  // namespace system
}  // namespace thrust
