// thrust::transform (unary and binary), thrust::for_each, thrust::sequence, thrust::gather,
// thrust::scatter: the element-wise callers on either side of the reduce / scan / sort path
// (thrust/system/detail/generic/transform.inl, sequence.inl, gather.inl, scatter.inl;
// thrust/system/cuda/detail/for_each.h).  On the device system they run as kernels that
// take the functor and the iterators by value, so they need a translation unit compiled
// with hipcc (functors __host__ __device__); the host system runs plain loops.
#pragma once
#include <algorithm>

#include <thrust/copy.h>
#include <thrust/iterator/counting_iterator.h>
#include <thrust/iterator/permutation_iterator.h>
#include <thrust/iterator/transform_iterator.h>
#include <thrust/iterator/zip_iterator.h>
#include <thrust/tuple.h>
#include <thrust/system/hip/detail/device_input.h>

namespace thrust {
namespace system {
namespace cpp {
template <typename D, typename In, typename Out, typename F>
Out transform(execution_policy<D>&, In first, In last, Out result, F f) {
  for (; first != last; ++first, ++result) *result = f(*first);
  return result;
}
template <typename D, typename In1, typename In2, typename Out, typename F>
Out transform(execution_policy<D>&, In1 first1, In1 last1, In2 first2, Out result, F f) {
  for (; first1 != last1; ++first1, ++first2, ++result) *result = f(*first1, *first2);
  return result;
}
template <typename D, typename It, typename F>
It for_each(execution_policy<D>&, It first, It last, F f) {
  for (; first != last; ++first) f(*first);
  return first;
}
template <typename D, typename It, typename T>
void sequence(execution_policy<D>&, It first, It last, T init, T step) {
  typedef typename iterator_value<It>::type V;
  for (std::size_t i = 0; first != last; ++first, ++i) *first = (V)(init + step * (T)i);
}
template <typename D, typename MapIt, typename In, typename Out>
Out gather(execution_policy<D>&, MapIt map_first, MapIt map_last, In input, Out result) {
  for (; map_first != map_last; ++map_first, ++result) *result = input[*map_first];
  return result;
}
template <typename D, typename In, typename MapIt, typename Out>
void scatter(execution_policy<D>&, In first, In last, MapIt map, Out output) {
  for (; first != last; ++first, ++map) output[*map] = *first;
}
}  // namespace cpp

namespace hip {
namespace detail {
template <typename T>
struct sequence_value {  // element i of thrust::sequence(first, last, init, step)
  T init, step;
  __host__ __device__ T operator()(unsigned long long i) const { return (T)(init + step * (T)i); }
};
}  // namespace detail

#if defined(__HIPCC__)
namespace detail {
// Arrays of 4- and 8-byte elements, suitably aligned, go through the kernels that move 16 bytes per
// access; everything else (fancy iterators, zips, other element sizes) through the plain ones.
template <typename ViewIn, typename ViewOut, typename F>
inline bool transform_packed(void*, ViewIn, ViewOut, uint64_t, F&) { return false; }
template <typename A, typename O, typename F>
inline typename std::enable_if<is_packable<typename std::remove_const<A>::type>::value && is_packable<O>::value &&
                                   !std::is_const<O>::value, bool>::type
transform_packed(void* stream, A* in, O* out, uint64_t n, F& f) {
  constexpr int PER = (sizeof(A) == 8 || sizeof(O) == 8) ? 2 : 4;
  if (n < 4096 || !pack_aligned(in, PER) || !pack_aligned(out, PER)) return false;
  hipLaunchKernelGGL((transform1_packed_kernel<A*, O, F, PER>), dim3(elementwise_grid(n / PER)), dim3(ELEMENTWISE_BLOCK),
                     0, (hipStream_t)stream, in, out, n, f);
  return true;
}
template <typename View, typename F>
inline bool for_each_packed(void*, View, uint64_t, F&) { return false; }
template <typename A, typename F>
inline typename std::enable_if<is_packable<typename std::remove_const<A>::type>::value, bool>::type
for_each_packed(void* stream, A* first, uint64_t n, F& f) {
  constexpr int PER = sizeof(A) == 8 ? 2 : 4;
  if (n < 4096 || !pack_aligned(first, PER)) return false;
  hipLaunchKernelGGL((for_each_packed_kernel<A*, F, PER>), dim3(elementwise_grid(n / PER)), dim3(ELEMENTWISE_BLOCK), 0,
                     (hipStream_t)stream, first, n, f);
  return true;
}
template <typename ViewA, typename ViewB, typename ViewOut, typename F>
inline bool transform_packed(void*, ViewA, ViewB, ViewOut, uint64_t, F&) { return false; }
template <typename A, typename B, typename O, typename F>
inline typename std::enable_if<is_packable<typename std::remove_const<A>::type>::value &&
                                   is_packable<typename std::remove_const<B>::type>::value && is_packable<O>::value &&
                                   !std::is_const<O>::value, bool>::type
transform_packed(void* stream, A* ina, B* inb, O* out, uint64_t n, F& f) {
  constexpr int PER = (sizeof(A) == 8 || sizeof(B) == 8 || sizeof(O) == 8) ? 2 : 4;
  if (n < 4096 || !pack_aligned(ina, PER) || !pack_aligned(inb, PER) || !pack_aligned(out, PER)) return false;
  hipLaunchKernelGGL((transform2_packed_kernel<A*, B*, O, F, PER>), dim3(elementwise_grid(n / PER)),
                     dim3(ELEMENTWISE_BLOCK), 0, (hipStream_t)stream, ina, inb, out, n, f);
  return true;
}
}  // namespace detail
#endif

template <typename D, typename In, typename Out, typename F>
Out transform(execution_policy<D>& exec, In first, In last, Out result, F f) {
  static_assert(detail::is_device_input<In>::value && detail::is_device_output<Out>::value,
                "thrust::transform on the device system reads device or fancy iterators and writes device memory");
  void* stream = detail::stream_of(exec);
  const uint64_t n = (uint64_t)(last - first);
  if (n == 0) return result;
#if defined(__HIPCC__)
  if (!detail::transform_packed(stream, thrust::detail::device_view(first), thrust::detail::device_view(result), n, f))
    hipLaunchKernelGGL((detail::transform1_kernel<typename thrust::detail::device_view_of<In>::type,
                                                  typename thrust::detail::device_view_of<Out>::type, F>),
                       dim3(detail::elementwise_grid(n)), dim3(detail::ELEMENTWISE_BLOCK), 0, (hipStream_t)stream,
                       thrust::detail::device_view(first), thrust::detail::device_view(result), n, f);
  detail::throw_on_error(detail::launch_status(), "transform: kernel launch");
  detail::synchronize(stream, "transform: synchronize");
#else
  static_assert(detail::fancy_needs_hipcc<F>::value,
                "thrust::transform on the device system runs the functor in a kernel; compile this translation unit with hipcc");
#endif
  return result + n;
}
template <typename D, typename In1, typename In2, typename Out, typename F>
Out transform(execution_policy<D>& exec, In1 first1, In1 last1, In2 first2, Out result, F f) {
  static_assert(detail::is_device_input<In1>::value && detail::is_device_input<In2>::value &&
                    detail::is_device_output<Out>::value,
                "thrust::transform on the device system reads device or fancy iterators and writes device memory");
  void* stream = detail::stream_of(exec);
  const uint64_t n = (uint64_t)(last1 - first1);
  if (n == 0) return result;
#if defined(__HIPCC__)
  if (!detail::transform_packed(stream, thrust::detail::device_view(first1), thrust::detail::device_view(first2),
                                thrust::detail::device_view(result), n, f))
    hipLaunchKernelGGL((detail::transform2_kernel<typename thrust::detail::device_view_of<In1>::type,
                                                  typename thrust::detail::device_view_of<In2>::type,
                                                  typename thrust::detail::device_view_of<Out>::type, F>),
                       dim3(detail::elementwise_grid(n)), dim3(detail::ELEMENTWISE_BLOCK), 0, (hipStream_t)stream,
                       thrust::detail::device_view(first1), thrust::detail::device_view(first2),
                       thrust::detail::device_view(result), n, f);
  detail::throw_on_error(detail::launch_status(), "transform: kernel launch");
  detail::synchronize(stream, "transform: synchronize");
#else
  static_assert(detail::fancy_needs_hipcc<F>::value,
                "thrust::transform on the device system runs the functor in a kernel; compile this translation unit with hipcc");
#endif
  return result + n;
}
template <typename D, typename It, typename F>
It for_each(execution_policy<D>& exec, It first, It last, F f) {
  // (something a kernel can read is enough: the functor of a for_each over counting_iterator
  // works through pointers of its own)
  static_assert(detail::is_device_output<It>::value || detail::is_device_input<It>::value,
                "thrust::for_each on the device system needs device_ptr / device_vector iterators, raw device pointers "
                "or fancy iterators over them");
  void* stream = detail::stream_of(exec);
  const uint64_t n = (uint64_t)(last - first);
  if (n == 0) return last;
#if defined(__HIPCC__)
  if (!detail::for_each_packed(stream, thrust::detail::device_view(first), n, f))
    hipLaunchKernelGGL((detail::for_each_kernel<typename thrust::detail::device_view_of<It>::type, F>),
                       dim3(detail::elementwise_grid(n)), dim3(detail::ELEMENTWISE_BLOCK), 0, (hipStream_t)stream,
                       thrust::detail::device_view(first), n, f);
  detail::throw_on_error(detail::launch_status(), "for_each: kernel launch");
  detail::synchronize(stream, "for_each: synchronize");
#else
  static_assert(detail::fancy_needs_hipcc<F>::value,
                "thrust::for_each on the device system runs the functor in a kernel; compile this translation unit with hipcc");
#endif
  return last;
}
namespace detail {
// an array of arithmetic elements of the type of init: the library's kernel (no hipcc needed)
template <typename D, typename It, typename T>
void sequence(execution_policy<D>& exec, It first, It last, T init, T step, std::true_type) {
  throw_on_error(thrust_amd_sequence(thrust::detail::raw(first), (uint64_t)(last - first), dtype_of<T>::value, &init,
                                     &step, stream_of(exec)),
                 "sequence failed");
  synchronize(stream_of(exec), "sequence: synchronize");
}
// anything else: the values are computed by a transform iterator and copied through the output
template <typename D, typename It, typename T>
void sequence(execution_policy<D>& exec, It first, It last, T init, T step, std::false_type) {
  const sequence_value<T> value = {init, step};
  thrust::counting_iterator<unsigned long long> zero(0);
  thrust::copy(exec, thrust::make_transform_iterator(zero, value),
               thrust::make_transform_iterator(zero + (last - first), value), first);
}
}  // namespace detail
template <typename D, typename It, typename T>
void sequence(execution_policy<D>& exec, It first, It last, T init, T step) {
  detail::sequence(exec, first, last, init, step,
                   std::integral_constant<bool, detail::is_abi_type<T>::value && detail::is_array_of<T, It>::value>());
}
template <typename D, typename MapIt, typename In, typename Out>
Out gather(execution_policy<D>& exec, MapIt map_first, MapIt map_last, In input, Out result) {
  return thrust::copy(exec, thrust::make_permutation_iterator(input, map_first),
                      thrust::make_permutation_iterator(input, map_last), result);
}
template <typename D, typename In, typename MapIt, typename Out>
void scatter(execution_policy<D>& exec, In first, In last, MapIt map, Out output) {
  static_assert(detail::is_device_input<In>::value && detail::is_device_input<MapIt>::value &&
                    detail::is_device_output<Out>::value,
                "thrust::scatter on the device system reads device or fancy iterators and writes device memory");
  void* stream = detail::stream_of(exec);
  const uint64_t n = (uint64_t)(last - first);
  if (n == 0) return;
#if defined(__HIPCC__)
  hipLaunchKernelGGL((detail::scatter_kernel<typename thrust::detail::device_view_of<In>::type,
                                             typename thrust::detail::device_view_of<MapIt>::type,
                                             typename thrust::detail::device_view_of<Out>::type>),
                     dim3(detail::elementwise_grid(n)), dim3(detail::ELEMENTWISE_BLOCK), 0, (hipStream_t)stream,
                     thrust::detail::device_view(first), thrust::detail::device_view(map),
                     thrust::detail::device_view(output), n);
  detail::throw_on_error(detail::launch_status(), "scatter: kernel launch");
  detail::synchronize(stream, "scatter: synchronize");
#else
  static_assert(detail::fancy_needs_hipcc<In>::value,
                "thrust::scatter on the device system runs as a kernel over the iterators; compile this translation unit with hipcc");
#endif
}
}  // namespace hip
}  // namespace system

// ------------------------------------------------------------------ entry points
template <typename D, typename In, typename Out, typename F>
Out transform(const detail::execution_policy_base<D>& exec, In first, In last, Out result, F f) {
  return transform(detail::derived_cast(detail::strip_const(exec)), first, last, result, f);
}
template <typename D, typename In1, typename In2, typename Out, typename F>
Out transform(const detail::execution_policy_base<D>& exec, In1 first1, In1 last1, In2 first2, Out result, F f) {
  return transform(detail::derived_cast(detail::strip_const(exec)), first1, last1, first2, result, f);
}
template <typename In, typename Out, typename F,
          typename = typename std::enable_if<!detail::is_execution_policy<In>::value>::type>
Out transform(In first, In last, Out result, F f) {
  return thrust::transform(detail::policy_for<Out>(), first, last, result, f);
}
template <typename In1, typename In2, typename Out, typename F,
          typename = typename std::enable_if<!detail::is_execution_policy<In1>::value>::type>
Out transform(In1 first1, In1 last1, In2 first2, Out result, F f) {
  return thrust::transform(detail::policy_for<Out>(), first1, last1, first2, result, f);
}

template <typename D, typename It, typename F>
It for_each(const detail::execution_policy_base<D>& exec, It first, It last, F f) {
  return for_each(detail::derived_cast(detail::strip_const(exec)), first, last, f);
}
template <typename It, typename F>
It for_each(It first, It last, F f) {
  return thrust::for_each(detail::policy_for<It>(), first, last, f);
}

template <typename D, typename It, typename T>
void sequence(const detail::execution_policy_base<D>& exec, It first, It last, T init, T step) {
  sequence(detail::derived_cast(detail::strip_const(exec)), first, last, init, step);
}
template <typename D, typename It, typename T>
void sequence(const detail::execution_policy_base<D>& exec, It first, It last, T init) {
  thrust::sequence(exec, first, last, init, T(1));
}
template <typename D, typename It>
void sequence(const detail::execution_policy_base<D>& exec, It first, It last) {
  typedef typename iterator_value<It>::type T;
  thrust::sequence(exec, first, last, T(0), T(1));
}
template <typename It>
void sequence(It first, It last) {
  thrust::sequence(detail::policy_for<It>(), first, last);
}
template <typename It, typename T, typename = typename std::enable_if<!detail::is_execution_policy<It>::value>::type>
void sequence(It first, It last, T init) {
  thrust::sequence(detail::policy_for<It>(), first, last, init);
}
template <typename It, typename T, typename = typename std::enable_if<!detail::is_execution_policy<It>::value>::type>
void sequence(It first, It last, T init, T step) {
  thrust::sequence(detail::policy_for<It>(), first, last, init, step);
}

template <typename D, typename MapIt, typename In, typename Out>
Out gather(const detail::execution_policy_base<D>& exec, MapIt map_first, MapIt map_last, In input, Out result) {
  return gather(detail::derived_cast(detail::strip_const(exec)), map_first, map_last, input, result);
}
template <typename MapIt, typename In, typename Out>
Out gather(MapIt map_first, MapIt map_last, In input, Out result) {
  return thrust::gather(detail::policy_for<Out>(), map_first, map_last, input, result);
}
template <typename D, typename In, typename MapIt, typename Out>
void scatter(const detail::execution_policy_base<D>& exec, In first, In last, MapIt map, Out output) {
  scatter(detail::derived_cast(detail::strip_const(exec)), first, last, map, output);
}
template <typename In, typename MapIt, typename Out>
void scatter(In first, In last, MapIt map, Out output) {
  thrust::scatter(detail::policy_for<Out>(), first, last, map, output);
}

// ------------------------------------------------------------------ the conditional forms
// transform_if, gather_if, scatter_if write an element only where the predicate holds for the input
// element (transform_if without a stencil) or for the stencil; for_each_n is for_each over a count
// (thrust/system/detail/generic/transform.inl:79-190, gather.inl:60-105, scatter.inl:48-96,
// for_each.h; testing/transform.cu, gather.cu, scatter.cu, for_each.cu).  All of them are one
// for_each over the zipped ranges, so they run on either system.
namespace detail {
template <typename Op, typename Pred>
struct writes_if {
  mutable Op op;  // a caller's functors need not be const-callable
  mutable Pred pred;
  // (input, output): the input decides
  template <typename A, typename O>
  __host__ __device__ void operator()(thrust::tuple<A, O> t) const {
    if (pred(thrust::get<0>(t))) thrust::get<1>(t) = op(thrust::get<0>(t));
  }
  // (input, stencil, output)
  template <typename A, typename S, typename O>
  __host__ __device__ void operator()(thrust::tuple<A, S, O> t) const {
    if (pred(thrust::get<1>(t))) thrust::get<2>(t) = op(thrust::get<0>(t));
  }
  // (input 1, input 2, stencil, output)
  template <typename A, typename B, typename S, typename O>
  __host__ __device__ void operator()(thrust::tuple<A, B, S, O> t) const {
    if (pred(thrust::get<2>(t))) thrust::get<3>(t) = op(thrust::get<0>(t), thrust::get<1>(t));
  }
};
struct passes_on {
  template <typename V>
  __host__ __device__ const V& operator()(const V& x) const { return x; }
};
struct is_nonzero {
  template <typename V>
  __host__ __device__ bool operator()(const V& x) const { return x ? true : false; }
};
}  // namespace detail

template <typename D, typename In, typename Out, typename Op, typename Pred>
Out transform_if(const detail::execution_policy_base<D>& exec, In first, In last, Out result, Op op, Pred pred) {
  const std::ptrdiff_t n = last - first;
  auto zipped = thrust::make_zip_iterator(thrust::make_tuple(first, result));
  const detail::writes_if<Op, Pred> f = {op, pred};
  thrust::for_each(exec, zipped, zipped + n, f);
  return result + n;
}
template <typename D, typename In, typename St, typename Out, typename Op, typename Pred>
Out transform_if(const detail::execution_policy_base<D>& exec, In first, In last, St stencil, Out result, Op op,
                 Pred pred) {
  const std::ptrdiff_t n = last - first;
  auto zipped = thrust::make_zip_iterator(thrust::make_tuple(first, stencil, result));
  const detail::writes_if<Op, Pred> f = {op, pred};
  thrust::for_each(exec, zipped, zipped + n, f);
  return result + n;
}
template <typename D, typename In1, typename In2, typename St, typename Out, typename Op, typename Pred>
Out transform_if(const detail::execution_policy_base<D>& exec, In1 first1, In1 last1, In2 first2, St stencil, Out result,
                 Op op, Pred pred) {
  const std::ptrdiff_t n = last1 - first1;
  auto zipped = thrust::make_zip_iterator(thrust::make_tuple(first1, first2, stencil, result));
  const detail::writes_if<Op, Pred> f = {op, pred};
  thrust::for_each(exec, zipped, zipped + n, f);
  return result + n;
}
template <typename In, typename Out, typename Op, typename Pred,
          typename = typename std::enable_if<!detail::is_execution_policy<In>::value>::type>
Out transform_if(In first, In last, Out result, Op op, Pred pred) {
  return thrust::transform_if(detail::policy_for<Out>(), first, last, result, op, pred);
}
template <typename In, typename St, typename Out, typename Op, typename Pred,
          typename = typename std::enable_if<!detail::is_execution_policy<In>::value>::type>
Out transform_if(In first, In last, St stencil, Out result, Op op, Pred pred) {
  return thrust::transform_if(detail::policy_for<Out>(), first, last, stencil, result, op, pred);
}
template <typename In1, typename In2, typename St, typename Out, typename Op, typename Pred,
          typename = typename std::enable_if<!detail::is_execution_policy<In1>::value>::type>
Out transform_if(In1 first1, In1 last1, In2 first2, St stencil, Out result, Op op, Pred pred) {
  return thrust::transform_if(detail::policy_for<Out>(), first1, last1, first2, stencil, result, op, pred);
}

template <typename D, typename MapIt, typename St, typename In, typename Out, typename Pred>
Out gather_if(const detail::execution_policy_base<D>& exec, MapIt map_first, MapIt map_last, St stencil, In input,
              Out result, Pred pred) {
  return thrust::transform_if(exec, thrust::make_permutation_iterator(input, map_first),
                              thrust::make_permutation_iterator(input, map_last), stencil, result, detail::passes_on(),
                              pred);
}
template <typename D, typename MapIt, typename St, typename In, typename Out>
Out gather_if(const detail::execution_policy_base<D>& exec, MapIt map_first, MapIt map_last, St stencil, In input,
              Out result) {
  return thrust::gather_if(exec, map_first, map_last, stencil, input, result, detail::is_nonzero());
}
template <typename MapIt, typename St, typename In, typename Out, typename Pred,
          typename = typename std::enable_if<!detail::is_execution_policy<MapIt>::value>::type>
Out gather_if(MapIt map_first, MapIt map_last, St stencil, In input, Out result, Pred pred) {
  return thrust::gather_if(detail::policy_for<Out>(), map_first, map_last, stencil, input, result, pred);
}
template <typename MapIt, typename St, typename In, typename Out,
          typename = typename std::enable_if<!detail::is_execution_policy<MapIt>::value>::type>
Out gather_if(MapIt map_first, MapIt map_last, St stencil, In input, Out result) {
  return thrust::gather_if(detail::policy_for<Out>(), map_first, map_last, stencil, input, result);
}

template <typename D, typename In, typename MapIt, typename St, typename Out, typename Pred>
void scatter_if(const detail::execution_policy_base<D>& exec, In first, In last, MapIt map, St stencil, Out output,
                Pred pred) {
  thrust::transform_if(exec, first, last, stencil, thrust::make_permutation_iterator(output, map), detail::passes_on(),
                       pred);
}
template <typename D, typename In, typename MapIt, typename St, typename Out>
void scatter_if(const detail::execution_policy_base<D>& exec, In first, In last, MapIt map, St stencil, Out output) {
  thrust::scatter_if(exec, first, last, map, stencil, output, detail::is_nonzero());
}
template <typename In, typename MapIt, typename St, typename Out, typename Pred,
          typename = typename std::enable_if<!detail::is_execution_policy<In>::value>::type>
void scatter_if(In first, In last, MapIt map, St stencil, Out output, Pred pred) {
  thrust::scatter_if(detail::policy_for<Out>(), first, last, map, stencil, output, pred);
}
template <typename In, typename MapIt, typename St, typename Out,
          typename = typename std::enable_if<!detail::is_execution_policy<In>::value>::type>
void scatter_if(In first, In last, MapIt map, St stencil, Out output) {
  thrust::scatter_if(detail::policy_for<Out>(), first, last, map, stencil, output);
}

template <typename D, typename It, typename Size, typename F>
It for_each_n(const detail::execution_policy_base<D>& exec, It first, Size n, F f) {
  return thrust::for_each(exec, first, first + (std::ptrdiff_t)n, f);
}
template <typename It, typename Size, typename F,
          typename = typename std::enable_if<!detail::is_execution_policy<It>::value>::type>
It for_each_n(It first, Size n, F f) {
  return thrust::for_each(detail::policy_for<It>(), first, first + (std::ptrdiff_t)n, f);
}

}  // namespace thrust
