// Inputs of the device system's algorithms.  device_ptr / device_vector iterators and raw
// device pointers are used where they lie.  A fancy iterator (counting, constant,
// transform, permutation) is written out into temporary storage first by a kernel that
// takes the iterator by value, and the algorithm then reads that array: the element is
// computed once per position, as the reference's load iterators do it
// (thrust/system/cuda/detail/core/util.h:527-561), at the price of one more write and
// read of the range.  That kernel is a template on the iterator, so fancy inputs need a
// translation unit compiled with hipcc.
#pragma once
#include <thrust/iterator/detail/fancy_iterator_base.h>
#include <thrust/iterator/permutation_iterator.h>
#include <thrust/iterator/reverse_iterator.h>
#include <thrust/iterator/zip_iterator.h>
#include <thrust/system/hip/detail/backend.h>
#if defined(__HIPCC__)
#include <thrust/system/hip/detail/fancy_kernels.h>
#endif

namespace thrust {
namespace system {
namespace hip {
namespace detail {

template <typename It>
struct is_device_input
    : std::integral_constant<bool, std::is_pointer<It>::value || thrust::detail::is_device_iterator<It>::value ||
                                       thrust::detail::is_fancy_iterator<It>::value> {};

// Where kernels that take iterators by value may write: device memory, or a zip of such.
template <typename It>
struct is_device_output
    : std::integral_constant<bool, std::is_pointer<It>::value || thrust::detail::is_device_iterator<It>::value ||
                                       thrust::detail::is_user_device_iterator<It>::value ||
                                       thrust::detail::is_fancy_output_iterator<It>::value> {};

template <>
struct is_device_output<thrust::zip_iterator<thrust::tuple<> > > : std::true_type {};
template <typename H, typename... T>
struct is_device_output<thrust::zip_iterator<thrust::tuple<H, T...> > >
    : std::integral_constant<bool, is_device_output<H>::value &&
                                       is_device_output<thrust::zip_iterator<thrust::tuple<T...> > >::value> {};

// a permutation of something writable, through indices that can be read
template <typename E, typename I>
struct is_device_output<thrust::permutation_iterator<E, I> >
    : std::integral_constant<bool, is_device_output<E>::value && is_device_input<I>::value> {};

// a range of something writable, walked backwards
template <typename It>
struct is_device_output<thrust::reverse_iterator<It> > : is_device_output<It> {};

template <typename It>
struct fancy_needs_hipcc : std::false_type {};

// Writes first[0, n) to out[0, n) (a device pointer, device_ptr or a zip of them) on the stream.
template <typename It, typename Out>
inline void materialize(void* stream, It first, Out out, uint64_t n) {
#if defined(__HIPCC__)
  if (n == 0) return;
  typedef typename thrust::detail::device_view_of<It>::type View;
  typedef typename thrust::detail::device_view_of<Out>::type OutView;
  hipLaunchKernelGGL((materialize_kernel<View, OutView>), dim3(elementwise_grid(n)), dim3(ELEMENTWISE_BLOCK), 0,
                     (hipStream_t)stream, thrust::detail::device_view(first), thrust::detail::device_view(out), n);
  throw_on_error(launch_status(), "fancy iterator: materialisation kernel");
#else
  static_assert(fancy_needs_hipcc<It>::value,
                "fancy iterators on the device system are read by kernels instantiated for the iterator; compile "
                "this translation unit with hipcc");
#endif
}

template <typename It, bool Fancy = thrust::detail::is_fancy_iterator<It>::value>
class device_input {
 public:
  typedef typename std::remove_const<typename iterator_value<It>::type>::type value_type;
  device_input(void*, const temp_source&, It first, uint64_t) : ptr_(thrust::detail::raw(first)) {}
  const value_type* ptr() const { return ptr_; }

 private:
  const value_type* ptr_;
};

template <typename It>
class device_input<It, true> {
 public:
  typedef typename std::remove_const<typename iterator_value<It>::type>::type value_type;
  device_input(void* stream, const temp_source& source, It first, uint64_t n) : holder_(stream, source), ptr_(nullptr) {
    if (n == 0) return;
    holder_.ensure((std::size_t)n * sizeof(value_type));
    ptr_ = static_cast<value_type*>(holder_.ptr());
    materialize(stream, first, ptr_, n);
  }
  const value_type* ptr() const { return ptr_; }

 private:
  temp_storage holder_;
  value_type* ptr_;
};

}  // namespace detail
}  // namespace hip
}  // namespace system
}  // namespace thrust
