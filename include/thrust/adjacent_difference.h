// thrust::adjacent_difference: result[0] = x[0], result[i] = x[i] - x[i-1] (or op(x[i], x[i-1]));
// the output may be the input (thrust/system/detail/generic/adjacent_difference.inl:35-78,
// thrust/system/cuda/detail/adjacent_difference.h; testing/adjacent_difference.cu).  On the device
// system: one binary transform over the range and itself shifted by one, from a copy of the input
// when the output is the input.
#pragma once
#include <cstddef>

#include <thrust/copy.h>
#include <thrust/device_vector.h>
#include <thrust/functional.h>
#include <thrust/host_vector.h>
#include <thrust/transform.h>

namespace thrust {

template <typename D, typename In, typename Out, typename Op>
Out adjacent_difference(const detail::execution_policy_base<D>& exec, In first, In last, Out result, Op op);

namespace system {
namespace cpp {
template <typename D, typename In, typename Out, typename Op>
Out adjacent_difference(execution_policy<D>&, In first, In last, Out result, Op op) {
  typedef typename std::remove_const<typename iterator_value<In>::type>::type V;
  if (first == last) return result;
  V previous = *first;
  *result = previous;
  for (++first, ++result; first != last; ++first, ++result) {
    const V current = *first;  // read before the write: the output may be the input
    *result = op(current, previous);
    previous = current;
  }
  return result;
}
}  // namespace cpp

namespace hip {
namespace detail {
template <typename A, typename B>
inline bool same_position(const A&, const B&) { return false; }
template <typename A>
inline bool same_position(const A& a, const A& b) { return a == b; }

// Whether writing n results from `out` on may change inputs that later results still read.  Two
// ranges in memory are compared by address, whatever their iterator types (a const iterator and
// a plain one of the same vector, a raw pointer and a device_ptr); other iterators by equality
// where they are of one type.
template <typename A, typename B>
inline bool output_reaches_input(A* in, B* out, std::size_t n) {
  const char* in_begin = reinterpret_cast<const char*>(in);
  const char* in_end = reinterpret_cast<const char*>(in + n);
  const char* out_begin = reinterpret_cast<const char*>(out);
  const char* out_end = reinterpret_cast<const char*>(out + n);
  return out_begin < in_end && in_begin < out_end;
}
template <typename ViewIn, typename ViewOut>
inline bool output_reaches_input(const ViewIn&, const ViewOut&, std::size_t) { return false; }

#if defined(__HIPCC__)
// arrays of 4- and 8-byte elements: one kernel that moves 16 bytes per access
template <typename ViewIn, typename ViewOut, typename Op>
inline bool adjacent_packed(void*, ViewIn, ViewOut, uint64_t, Op&) { return false; }
template <typename A, typename O, typename Op>
inline typename std::enable_if<is_packable<typename std::remove_const<A>::type>::value && is_packable<O>::value &&
                                   !std::is_const<O>::value, bool>::type
adjacent_packed(void* stream, A* in, O* out, uint64_t n, Op& op) {
  constexpr int PER = (sizeof(A) == 8 || sizeof(O) == 8) ? 2 : 4;
  if (n < 4096 || !pack_aligned(in, PER) || !pack_aligned(out, PER)) return false;
  hipLaunchKernelGGL((adjacent_packed_kernel<typename std::remove_const<A>::type, O, Op, PER>),
                     dim3(elementwise_grid(n / PER)), dim3(ELEMENTWISE_BLOCK), 0, (hipStream_t)stream, in, out, n, op);
  return true;
}
#endif
}  // namespace detail

template <typename D, typename In, typename Out, typename Op>
Out adjacent_difference(execution_policy<D>& exec, In first, In last, Out result, Op op) {
  typedef typename std::remove_const<typename iterator_value<In>::type>::type V;
  const std::ptrdiff_t n = last - first;
  if (n == 0) return result;
  if (detail::same_position(first, result) ||
      detail::output_reaches_input(thrust::detail::device_view(first), thrust::detail::device_view(result), (std::size_t)n)) {
    thrust::device_vector<V> input(first, last);
    return thrust::adjacent_difference(exec, input.begin(), input.end(), result, op);
  }
#if defined(__HIPCC__)
  if (detail::adjacent_packed(detail::stream_of(exec), thrust::detail::device_view(first),
                              thrust::detail::device_view(result), (uint64_t)n, op)) {
    detail::throw_on_error(detail::launch_status(), "adjacent_difference: kernel launch");
    detail::synchronize(detail::stream_of(exec), "adjacent_difference: synchronize");
    return result + n;
  }
#endif
  thrust::copy(exec, first, first + 1, result);
  thrust::transform(exec, first + 1, last, first, result + 1, op);
  return result + n;
}
}  // namespace hip
}  // namespace system

template <typename D, typename In, typename Out, typename Op>
Out adjacent_difference(const detail::execution_policy_base<D>& exec, In first, In last, Out result, Op op) {
  return adjacent_difference(detail::derived_cast(detail::strip_const(exec)), first, last, result, op);
}
template <typename D, typename In, typename Out>
Out adjacent_difference(const detail::execution_policy_base<D>& exec, In first, In last, Out result) {
  typedef typename std::remove_const<typename iterator_value<In>::type>::type V;
  return thrust::adjacent_difference(exec, first, last, result, thrust::minus<V>());
}
template <typename In, typename Out, typename Op,
          typename = typename std::enable_if<!detail::is_execution_policy<In>::value>::type>
Out adjacent_difference(In first, In last, Out result, Op op) {
  return thrust::adjacent_difference(detail::policy_for<Out>(), first, last, result, op);
}
template <typename In, typename Out>
Out adjacent_difference(In first, In last, Out result) {
  return thrust::adjacent_difference(detail::policy_for<Out>(), first, last, result);
}

}  // namespace thrust
