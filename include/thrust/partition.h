// thrust::partition, stable_partition, partition_copy, stable_partition_copy (with and
// without stencil).
//
// All four are stable here, as in the reference's generic layer where partition is
// stable_partition (thrust/system/detail/generic/partition.inl:46-64,103-119,154-160).
// On the device system the predicate must be one of the recognised forms listed in
// thrust/functional.h.
#pragma once
#include <algorithm>
#include <vector>

#include <thrust/copy.h>
#include <thrust/logical.h>
#include <thrust/pair.h>

namespace thrust {

namespace system {
namespace cpp {
template <typename D, typename It, typename St, typename Pred>
It stable_partition(execution_policy<D>&, It first, It last, St stencil, Pred pred) {
  typedef typename iterator_value<It>::type T;
  std::vector<T> yes, no;
  for (It it = first; it != last; ++it, ++stencil) (pred(*stencil) ? yes : no).push_back(*it);
  It mid = std::copy(yes.begin(), yes.end(), first);
  std::copy(no.begin(), no.end(), mid);
  return mid;
}
template <typename D, typename It, typename Pred>
It stable_partition(execution_policy<D>& exec, It first, It last, Pred pred) {
  typedef typename iterator_value<It>::type T;
  std::vector<T> copy(first, last);
  return stable_partition(exec, first, last, copy.begin(), pred);
}
template <typename D, typename In, typename St, typename Out1, typename Out2, typename Pred>
pair<Out1, Out2> stable_partition_copy(execution_policy<D>&, In first, In last, St stencil, Out1 out_true,
                                       Out2 out_false, Pred pred) {
  for (; first != last; ++first, ++stencil) {
    if (pred(*stencil)) { *out_true = *first; ++out_true; }
    else { *out_false = *first; ++out_false; }
  }
  return thrust::make_pair(out_true, out_false);
}
template <typename D, typename In, typename Out1, typename Out2, typename Pred>
pair<Out1, Out2> stable_partition_copy(execution_policy<D>& exec, In first, In last, Out1 out_true, Out2 out_false,
                                       Pred pred) {
  return stable_partition_copy(exec, first, last, first, out_true, out_false, pred);
}
}  // namespace cpp

namespace hip {
namespace detail {
#if defined(__HIPCC__)
// a user's predicate: it runs inside the compaction kernel, instantiated here
template <typename D, typename It, typename St, typename HasStencil, typename Pred>
It stable_partition_impl(execution_policy<D>& exec, It first, It last, St stencil, HasStencil, Pred pred,
                         std::integral_constant<int, 1>) {
  typedef typename iterator_value<It>::type T;
  typedef typename std::remove_const<typename iterator_value<St>::type>::type S;
  static_assert(is_abi_item<T>::value, "stable_partition on the device system: items of 1, 2, 4 or 8 bytes");
  void* stream = stream_of(exec);
  const uint64_t n = (uint64_t)(last - first);
  if (n == 0) return first;
  device_input<St> tested(stream, temp_source_of(exec), stencil, HasStencil::value ? n : 0);
  T* data = thrust::detail::raw(first);
  const uint64_t cnt = generic_selection<HasStencil::value>(stream, temp_source_of(exec), (const T*)data,
                                                            (const S*)tested.ptr(), data, (T*)nullptr, true, n, pred,
                                                            false, "stable_partition failed");
  synchronize(stream, "stable_partition: synchronize");
  return first + cnt;
}
template <typename D, typename In, typename St, typename HasStencil, typename Out1, typename Out2, typename Pred>
pair<Out1, Out2> stable_partition_copy_impl(execution_policy<D>& exec, In first, In last, St stencil, HasStencil,
                                            Out1 out_true, Out2 out_false, Pred pred, std::integral_constant<int, 1>) {
  typedef typename std::remove_const<typename iterator_value<In>::type>::type T;
  typedef typename std::remove_const<typename iterator_value<St>::type>::type S;
  static_assert(is_abi_item<T>::value && std::is_same<typename iterator_value<Out1>::type, T>::value &&
                    std::is_same<typename iterator_value<Out2>::type, T>::value,
                "partition_copy on the device system: items of 1, 2, 4 or 8 bytes, same type in and out");
  void* stream = stream_of(exec);
  const uint64_t n = (uint64_t)(last - first);
  if (n == 0) return thrust::make_pair(out_true, out_false);
  device_input<In> source(stream, temp_source_of(exec), first, n);
  device_input<St> tested(stream, temp_source_of(exec), stencil, HasStencil::value ? n : 0);
  const uint64_t cnt = generic_selection<HasStencil::value>(
      stream, temp_source_of(exec), (const T*)source.ptr(), (const S*)tested.ptr(), thrust::detail::raw(out_true),
      thrust::detail::raw(out_false), false, n, pred, false, "partition_copy failed");
  synchronize(stream, "partition_copy: synchronize");
  return thrust::make_pair(out_true + cnt, out_false + (n - cnt));
}
#endif
template <typename D, typename It, typename St, typename HasStencil, typename Pred, int ROUTE>
It stable_partition_impl(execution_policy<D>& exec, It first, It last, St stencil, HasStencil, Pred pred,
                         std::integral_constant<int, ROUTE>) {
  typedef typename iterator_value<It>::type T;
  static_assert(is_abi_item<T>::value, "stable_partition on the device system: items of 1, 2, 4 or 8 bytes");
  const bool has_stencil = HasStencil::value;
  void* stream = stream_of(exec);
  const uint64_t n = (uint64_t)(last - first);
  if (n == 0) return first;
  tested_stream<St, Pred> tested(stream, temp_source_of(exec), stencil, n, pred, has_stencil);
  const uint64_t cnt = run_selection<typename tested_stream<St, Pred>::tested_type>(
      stream, temp_source_of(exec), tested.predicate(), "stable_partition failed",
      [&](void* t, std::size_t* b, uint64_t* d_num, int cmp, const void* thr) {
        return thrust_amd_stable_partition(t, b, thrust::detail::raw(first), tested.stencil(), d_num, n, sizeof(T),
                                           tested.dtype(), cmp, thr, stream);
      });
  synchronize(stream, "stable_partition: synchronize");
  return first + cnt;
}
template <typename D, typename In, typename St, typename HasStencil, typename Out1, typename Out2, typename Pred,
          int ROUTE>
pair<Out1, Out2> stable_partition_copy_impl(execution_policy<D>& exec, In first, In last, St stencil, HasStencil,
                                            Out1 out_true, Out2 out_false, Pred pred,
                                            std::integral_constant<int, ROUTE>) {
  const bool has_stencil = HasStencil::value;
  typedef typename std::remove_const<typename iterator_value<In>::type>::type T;
  static_assert(is_abi_item<T>::value && std::is_same<typename iterator_value<Out1>::type, T>::value &&
                    std::is_same<typename iterator_value<Out2>::type, T>::value,
                "partition_copy on the device system: items of 1, 2, 4 or 8 bytes, same type in and out");
  void* stream = stream_of(exec);
  const uint64_t n = (uint64_t)(last - first);
  if (n == 0) return thrust::make_pair(out_true, out_false);
  device_input<In> source(stream, temp_source_of(exec), first, n);
  tested_stream<St, Pred> tested(stream, temp_source_of(exec), stencil, n, pred, has_stencil);
  const uint64_t cnt = run_selection<typename tested_stream<St, Pred>::tested_type>(
      stream, temp_source_of(exec), tested.predicate(), "partition_copy failed",
      [&](void* t, std::size_t* b, uint64_t* d_num, int cmp, const void* thr) {
        return thrust_amd_partition_copy(t, b, source.ptr(), tested.stencil(), thrust::detail::raw(out_true),
                                         thrust::detail::raw(out_false), d_num, n, sizeof(T), tested.dtype(), cmp, thr,
                                         stream);
      });
  synchronize(stream, "partition_copy: synchronize");
  return thrust::make_pair(out_true + cnt, out_false + (n - cnt));
}
template <typename D, typename It, typename St, typename HasStencil, typename Pred>
It stable_partition_impl(execution_policy<D>& exec, It first, It last, St stencil, HasStencil has_stencil, Pred pred) {
  typedef typename std::remove_const<typename iterator_value<St>::type>::type S;
  return stable_partition_impl(exec, first, last, stencil, has_stencil, pred, selection_route<Pred, S>());
}
template <typename D, typename In, typename St, typename HasStencil, typename Out1, typename Out2, typename Pred>
pair<Out1, Out2> stable_partition_copy_impl(execution_policy<D>& exec, In first, In last, St stencil,
                                            HasStencil has_stencil, Out1 out_true, Out2 out_false, Pred pred) {
  typedef typename std::remove_const<typename iterator_value<St>::type>::type S;
  return stable_partition_copy_impl(exec, first, last, stencil, has_stencil, out_true, out_false, pred,
                                    selection_route<Pred, S>());
}
}  // namespace detail

namespace detail {
// Items of 1, 2, 4 or 8 bytes in arrays of one type: the compaction kernels.  Anything else
// (wider elements, zip or discard iterators, another output type): the three-pass selection
// through the iterators themselves.
template <typename D, typename It, typename St, typename HasStencil, typename Pred>
It stable_partition_any(execution_policy<D>& exec, It first, It last, St stencil, HasStencil has_stencil, Pred pred,
                        std::true_type) {
  return stable_partition_impl(exec, first, last, stencil, has_stencil, pred);
}
template <typename D, typename In, typename St, typename HasStencil, typename Out1, typename Out2, typename Pred>
pair<Out1, Out2> stable_partition_copy_any(execution_policy<D>& exec, In first, In last, St stencil,
                                           HasStencil has_stencil, Out1 out_true, Out2 out_false, Pred pred,
                                           std::true_type) {
  return stable_partition_copy_impl(exec, first, last, stencil, has_stencil, out_true, out_false, pred);
}
template <typename D, typename It, typename St, typename HasStencil, typename Pred>
It stable_partition_any(execution_policy<D>& exec, It first, It last, St stencil, HasStencil, Pred pred,
                        std::false_type) {
#if defined(__HIPCC__)
  return first + partition_any_range(exec, first, (uint64_t)(last - first), stencil, pred, "stable_partition failed");
#else
  static_assert(fancy_needs_hipcc<Pred>::value,
                "thrust::partition / stable_partition on the device system: items other than 1, 2, 4 or 8 bytes and "
                "ranges that are not arrays are handled by kernels instantiated for the iterators; compile this "
                "translation unit with hipcc");
  return first;
#endif
}
template <typename D, typename In, typename St, typename HasStencil, typename Out1, typename Out2, typename Pred>
pair<Out1, Out2> stable_partition_copy_any(execution_policy<D>& exec, In first, In last, St stencil, HasStencil,
                                           Out1 out_true, Out2 out_false, Pred pred, std::false_type) {
#if defined(__HIPCC__)
  const uint64_t n = (uint64_t)(last - first);
  const uint64_t cnt = select_any_range<true>(exec, first, n, stencil, out_true, out_false, pred, false,
                                              "partition_copy failed");
  return thrust::make_pair(out_true + cnt, out_false + (n - cnt));
#else
  static_assert(fancy_needs_hipcc<Pred>::value,
                "thrust::partition_copy / stable_partition_copy on the device system: items other than 1, 2, 4 or 8 "
                "bytes and outputs that are not arrays of the input's type are handled by kernels instantiated for "
                "the iterators; compile this translation unit with hipcc");
  return thrust::make_pair(out_true, out_false);
#endif
}
template <typename D, typename It, typename St, typename HasStencil, typename Pred>
It stable_partition_any(execution_policy<D>& exec, It first, It last, St stencil, HasStencil has_stencil, Pred pred) {
  typedef typename std::remove_const<typename iterator_value<It>::type>::type T;
  return stable_partition_any(exec, first, last, stencil, has_stencil, pred,
                              std::integral_constant<bool, is_abi_item<T>::value && is_array_of<T, It>::value>());
}
template <typename D, typename In, typename St, typename HasStencil, typename Out1, typename Out2, typename Pred>
pair<Out1, Out2> stable_partition_copy_any(execution_policy<D>& exec, In first, In last, St stencil,
                                           HasStencil has_stencil, Out1 out_true, Out2 out_false, Pred pred) {
  typedef typename std::remove_const<typename iterator_value<In>::type>::type T;
  return stable_partition_copy_any(
      exec, first, last, stencil, has_stencil, out_true, out_false, pred,
      std::integral_constant<bool, is_abi_item<T>::value && is_array_of<T, Out1>::value && is_array_of<T, Out2>::value>());
}
}  // namespace detail

template <typename D, typename It, typename Pred>
It stable_partition(execution_policy<D>& exec, It first, It last, Pred pred) {
  return detail::stable_partition_any(exec, first, last, first, std::false_type(), pred);
}
template <typename D, typename It, typename St, typename Pred>
It stable_partition(execution_policy<D>& exec, It first, It last, St stencil, Pred pred) {
  return detail::stable_partition_any(exec, first, last, stencil, std::true_type(), pred);
}
template <typename D, typename In, typename Out1, typename Out2, typename Pred>
pair<Out1, Out2> stable_partition_copy(execution_policy<D>& exec, In first, In last, Out1 out_true, Out2 out_false,
                                       Pred pred) {
  return detail::stable_partition_copy_any(exec, first, last, first, std::false_type(), out_true, out_false, pred);
}
template <typename D, typename In, typename St, typename Out1, typename Out2, typename Pred>
pair<Out1, Out2> stable_partition_copy(execution_policy<D>& exec, In first, In last, St stencil, Out1 out_true,
                                       Out2 out_false, Pred pred) {
  return detail::stable_partition_copy_any(exec, first, last, stencil, std::true_type(), out_true, out_false, pred);
}
}  // namespace hip
}  // namespace system

// ------------------------------------------------------------------ entry points
// partition == stable_partition, partition_copy == stable_partition_copy
// (thrust/system/detail/generic/partition.inl:154-160,196-214).
#define THRUST_AMD_PARTITION_ENTRY(NAME)                                                                        \
  template <typename D, typename It, typename Pred>                                                             \
  It NAME(const detail::execution_policy_base<D>& exec, It first, It last, Pred pred) {                         \
    return stable_partition(detail::derived_cast(detail::strip_const(exec)), first, last, pred);                \
  }                                                                                                             \
  template <typename D, typename It, typename St, typename Pred>                                                \
  It NAME(const detail::execution_policy_base<D>& exec, It first, It last, St stencil, Pred pred) {             \
    return stable_partition(detail::derived_cast(detail::strip_const(exec)), first, last, stencil, pred);       \
  }                                                                                                             \
  template <typename It, typename Pred>                                                                         \
  It NAME(It first, It last, Pred pred) { return thrust::NAME(detail::policy_for<It>(), first, last, pred); }   \
  template <typename It, typename St, typename Pred,                                                            \
            typename = typename std::enable_if<!detail::is_execution_policy<It>::value>::type>                  \
  It NAME(It first, It last, St stencil, Pred pred) {                                                           \
    return thrust::NAME(detail::policy_for<It>(), first, last, stencil, pred);                                  \
  }
THRUST_AMD_PARTITION_ENTRY(partition)
THRUST_AMD_PARTITION_ENTRY(stable_partition)
#undef THRUST_AMD_PARTITION_ENTRY

#define THRUST_AMD_PARTITION_COPY_ENTRY(NAME)                                                                   \
  template <typename D, typename In, typename Out1, typename Out2, typename Pred>                               \
  pair<Out1, Out2> NAME(const detail::execution_policy_base<D>& exec, In first, In last, Out1 out_true,         \
                        Out2 out_false, Pred pred) {                                                            \
    return stable_partition_copy(detail::derived_cast(detail::strip_const(exec)), first, last, out_true,        \
                                 out_false, pred);                                                              \
  }                                                                                                             \
  template <typename D, typename In, typename St, typename Out1, typename Out2, typename Pred>                  \
  pair<Out1, Out2> NAME(const detail::execution_policy_base<D>& exec, In first, In last, St stencil,            \
                        Out1 out_true, Out2 out_false, Pred pred) {                                             \
    return stable_partition_copy(detail::derived_cast(detail::strip_const(exec)), first, last, stencil,         \
                                 out_true, out_false, pred);                                                    \
  }                                                                                                             \
  template <typename In, typename Out1, typename Out2, typename Pred>                                           \
  pair<Out1, Out2> NAME(In first, In last, Out1 out_true, Out2 out_false, Pred pred) {                          \
    return thrust::NAME(detail::policy_for<In>(), first, last, out_true, out_false, pred);                      \
  }                                                                                                             \
  template <typename In, typename St, typename Out1, typename Out2, typename Pred,                              \
            typename = typename std::enable_if<!detail::is_execution_policy<In>::value>::type>                  \
  pair<Out1, Out2> NAME(In first, In last, St stencil, Out1 out_true, Out2 out_false, Pred pred) {              \
    return thrust::NAME(detail::policy_for<In>(), first, last, stencil, out_true, out_false, pred);             \
  }
THRUST_AMD_PARTITION_COPY_ENTRY(partition_copy)
THRUST_AMD_PARTITION_COPY_ENTRY(stable_partition_copy)
#undef THRUST_AMD_PARTITION_COPY_ENTRY

// ------------------------------------------------------------------ is_partitioned, partition_point
// partition_point: the end of the leading elements that satisfy the predicate, for a range that is
// partitioned by it; is_partitioned: no element after that point satisfies it
// (thrust/system/detail/generic/partition.inl:163-214; testing/partition_point.cu, is_partitioned.cu).
template <typename D, typename It, typename Pred>
It partition_point(const detail::execution_policy_base<D>& exec, It first, It last, Pred pred) {
  return thrust::find_if_not(exec, first, last, pred);
}
template <typename It, typename Pred, typename = typename std::enable_if<!detail::is_execution_policy<It>::value>::type>
It partition_point(It first, It last, Pred pred) {
  return thrust::partition_point(detail::policy_for<It>(), first, last, pred);
}
template <typename D, typename It, typename Pred>
bool is_partitioned(const detail::execution_policy_base<D>& exec, It first, It last, Pred pred) {
  const It mid = thrust::find_if_not(exec, first, last, pred);
  if (mid == last) return true;
  return thrust::none_of(exec, mid + 1, last, pred);
}
template <typename It, typename Pred, typename = typename std::enable_if<!detail::is_execution_policy<It>::value>::type>
bool is_partitioned(It first, It last, Pred pred) {
  return thrust::is_partitioned(detail::policy_for<It>(), first, last, pred);
}

}  // namespace thrust
