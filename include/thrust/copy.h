// thrust::copy, thrust::copy_n and thrust::copy_if.
//
// copy moves trivially copyable elements inside one system or across the two
// (the reference: thrust/system/cuda/detail/internal/copy_cross_system.h:50-200,
// util.h:107-162).  copy_if is a stable compaction, with or without a stencil
// (thrust/system/detail/generic/copy_if.inl:97-154); on the device system the predicate
// must be one of the recognised forms listed in thrust/functional.h.
#pragma once
#include <algorithm>
#include <vector>

#include <thrust/host_vector.h>
#include <thrust/functional.h>
#include <thrust/iterator/transform_iterator.h>
#include <thrust/system/hip/detail/backend.h>
#include <thrust/system/hip/detail/device_input.h>
#include <thrust/system/hip/detail/staged_output.h>
#if defined(__HIPCC__)
#include <thrust/system/hip/detail/generic_select.h>
#include <thrust/system/hip/detail/any_range_selection.h>
#endif

namespace thrust {

namespace detail {
// Copy n elements between any two of {host, device} given raw element addresses.
template <typename T>
inline void copy_raw(const T* src, bool src_device, T* dst, bool dst_device, std::size_t n, void* stream,
                     bool blocking = true) {
  if (n == 0) return;
  using thrust::system::hip::detail::throw_on_error;
  if (!src_device && !dst_device) {
    std::copy(src, src + n, dst);
  } else if (src_device && dst_device) {
    throw_on_error(thrust_amd_memcpy(dst, src, n * sizeof(T), THRUST_AMD_D2D, stream), "copy (device to device)");
    if (blocking) throw_on_error(thrust_amd_stream_synchronize(stream), "copy: synchronize");
  } else {
    throw_on_error(thrust_amd_memcpy(dst, src, n * sizeof(T), src_device ? THRUST_AMD_D2H : THRUST_AMD_H2D, stream),
                   "copy (across systems)");
  }
}

// result + n for the iterators that were written through their address
template <typename Out>
inline Out advanced(Out result, std::size_t n, std::true_type) { return result + n; }
template <typename Out>
inline Out advanced(Out result, std::size_t, std::false_type) { return result; }

// Fancy iterators have no address: element by element through the iterators themselves
// (host code; device_ptr ends go through their host-side proxies).
template <typename In, typename Out>
inline typename std::enable_if<is_fancy_iterator<In>::value || is_fancy_iterator<Out>::value, Out>::type copy_dispatch(
    In first, In last, Out result, bool, bool, void*, bool = true) {
  for (; first != last; ++first, ++result) *result = *first;
  return result;
}
template <typename In, typename Out>
inline typename std::enable_if<!is_fancy_iterator<In>::value && !is_fancy_iterator<Out>::value, Out>::type copy_dispatch(
    In first, In last, Out result, bool in_device, bool out_device, void* stream, bool blocking = true) {
  typedef typename std::remove_const<typename iterator_value<In>::type>::type T;
  // (pure output iterators such as std::back_insert_iterator name no value type)
  typedef typename std::conditional<std::is_void<typename iterator_value<Out>::type>::value, T,
                                    typename iterator_value<Out>::type>::type U;
  const std::size_t n = (std::size_t)std::distance(first, last);
  if (n == 0) return result;
  if (!in_device && !out_device) return std::copy(first, last, result);
  static_assert(std::is_trivially_copy_constructible<T>::value,
                "thrust::copy involving the device needs trivially copy-constructible elements");
  // addresses of the ends that have one (a device end always has)
  typedef std::integral_constant<bool, is_device_iterator<In>::value || std::is_pointer<In>::value ||
                                           is_contiguous_host_iterator<In>::value> in_has_address;
  typedef std::integral_constant<bool, is_device_iterator<Out>::value || std::is_pointer<Out>::value ||
                                           is_contiguous_host_iterator<Out>::value> out_has_address;
  const T* in_raw = raw_if<const T>(first, in_has_address());
  U* out_raw = raw_if<U>(result, out_has_address());
  if (std::is_same<T, U>::value && (in_device || is_contiguous_host_iterator<In>::value) &&
      (out_device || is_contiguous_host_iterator<Out>::value)) {
    copy_raw<T>(in_raw, in_device, reinterpret_cast<T*>(out_raw), out_device, n, stream, blocking);
  } else if (in_device) {
    // device -> host with conversion or a non-contiguous destination: stage on the host
    staging_vector<T> staged(n);
    copy_raw<T>(in_raw, true, staged.data(), false, n, stream);
    if (out_device) {
      staging_vector<U> converted(staged.begin(), staged.end());
      copy_raw<U>(converted.data(), false, out_raw, true, n, stream);
    } else {
      return std::copy(staged.begin(), staged.end(), result);
    }
  } else {
    staging_vector<U> staged(first, last);
    copy_raw<U>(staged.data(), false, out_raw, true, n, stream);
  }
  return advanced(result, n, out_has_address());
}
}  // namespace detail

template <typename D, typename In, typename Out, typename Pred>
Out copy_if(const detail::execution_policy_base<D>& exec, In first, In last, Out result, Pred pred);
template <typename D, typename In, typename St, typename Out, typename Pred>
Out copy_if(const detail::execution_policy_base<D>& exec, In first, In last, St stencil, Out result, Pred pred);

namespace system {
namespace cpp {
template <typename D, typename In, typename Out>
Out copy(execution_policy<D>&, In first, In last, Out result) {
  return thrust::detail::copy_dispatch(first, last, result, thrust::detail::is_device_iterator<In>::value,
                                       thrust::detail::is_device_iterator<Out>::value, nullptr);
}
template <typename D, typename In, typename St, typename Out, typename Pred>
Out copy_if(execution_policy<D>&, In first, In last, St stencil, Out result, Pred pred) {
  for (; first != last; ++first, ++stencil)
    if (pred(*stencil)) { *result = *first; ++result; }
  return result;
}
template <typename D, typename In, typename Out, typename Pred>
Out copy_if(execution_policy<D>& exec, In first, In last, Out result, Pred pred) {
  return copy_if(exec, first, last, first, result, pred);
}
}  // namespace cpp

namespace hip {
namespace detail {
template <typename D, typename In, typename Out>
Out copy(execution_policy<D>& exec, In first, In last, Out result, std::false_type) {
  // explicit device policy: raw pointers are device pointers
  const bool in_dev = thrust::detail::is_device_iterator<In>::value || std::is_pointer<In>::value;
  const bool out_dev = thrust::detail::is_device_iterator<Out>::value || std::is_pointer<Out>::value;
  return thrust::detail::copy_dispatch(first, last, result, in_dev, out_dev, stream_of(exec));
}
// from a fancy iterator to device memory: the materialisation kernel writes straight into
// the destination; to host memory: the iterator is walked on the host
template <typename D, typename In, typename Out>
Out copy_fancy(execution_policy<D>& exec, In first, In last, Out result, std::true_type) {
  void* stream = stream_of(exec);
  const uint64_t n = (uint64_t)(last - first);
  materialize(stream, first, result, n);
  synchronize(stream, "copy: synchronize");
  return result + n;
}
template <typename D, typename In, typename Out>
Out copy_fancy(execution_policy<D>&, In first, In last, Out result, std::false_type) {
  for (; first != last; ++first, ++result) *result = *first;
  return result;
}
template <typename D, typename In, typename Out>
Out copy(execution_policy<D>& exec, In first, In last, Out result, std::true_type) {
  // both ends on the device side: one kernel; otherwise the iterators are walked on the host
  return copy_fancy(exec, first, last, result,
                    std::integral_constant<bool, is_device_input<In>::value && is_device_output<Out>::value>());
}
// a user predicate as one byte per element, for the stencil form of the selection kernels
template <typename Pred>
struct as_flag {
  mutable Pred pred;  // a caller's predicate need not be const-callable
  template <typename V>
  __host__ __device__ unsigned char operator()(const V& x) const { return pred(x) ? 1 : 0; }
};
template <typename Pred, typename T, bool = is_abi_type<T>::value>
struct selects_in_kernel : std::integral_constant<bool, unary_pred<Pred, T>::supported> {};
template <typename Pred, typename T>
struct selects_in_kernel<Pred, T, false> : std::false_type {};
// 0: a recognised predicate, evaluated by the library's kernel from a comparison code
// 1: any other predicate on a type the compaction kernel can hold: the kernel is instantiated
//    for the predicate in this translation unit (hipcc) and evaluates it in registers
// 2: the predicate is evaluated into one byte per element first (tested types of other sizes)
template <typename Pred, typename S>
struct selection_route
    : std::integral_constant<int, selects_in_kernel<Pred, S>::value ? 0
#if defined(__HIPCC__)
                                  : is_kernel_item<S>::value ? 1
#endif
                                                             : 2> {};
}  // namespace detail

template <typename D, typename In, typename Out>
Out copy(execution_policy<D>& exec, In first, In last, Out result) {
  return detail::copy(exec, first, last, result,
                      std::integral_constant<bool, thrust::detail::is_fancy_iterator<In>::value ||
                                                       thrust::detail::is_fancy_iterator<Out>::value>());
}

namespace detail {
// Shared by copy_if and the partition family: runs `entry` (one of the three selection
// entry points bound by the caller) and returns the number of selected elements.
// `negate` selects the elements the predicate rejects (remove_if is copy_if of not1(pred),
// thrust/system/cuda/detail/remove.h:40-66).  The kernel evaluates the predicate and inverts
// the result; swapping in the complementary comparison would drop NaNs, which fail both.
inline int negated_cmp(int cmp) { return cmp ^ THRUST_AMD_CMP_NOT; }
template <typename Tested, typename Pred, typename Call>
inline uint64_t run_selection(void* stream, const temp_source& source, const Pred& pred, const char* what, Call call,
                              bool negate = false) {
  static_assert(is_abi_type<Tested>::value,
                "selection on the device system needs an arithmetic type to test");
  static_assert(unary_pred<Pred, Tested>::supported,
                "selection on the device system supports placeholder comparisons (_1 < t, ...), "
                "thrust::identity and thrust::logical_not as predicate");
  const int cmp = negate ? negated_cmp(unary_pred<Pred, Tested>::cmp(pred)) : unary_pred<Pred, Tested>::cmp(pred);
  const Tested thr = unary_pred<Pred, Tested>::threshold(pred);
  temp_storage temp(stream, source);
  std::size_t need = 0;
  uint64_t* d_num = nullptr;
  throw_on_error(call((void*)nullptr, &need, d_num, cmp, (const void*)&thr), what);
  const std::size_t aligned = (need + 255) / 256 * 256;
  temp.ensure(aligned + 256);
  d_num = reinterpret_cast<uint64_t*>(static_cast<char*>(temp.ptr()) + aligned);
  std::size_t bytes = aligned;
  throw_on_error(call(temp.ptr(), &bytes, d_num, cmp, (const void*)&thr), what);
  return read_scalar<uint64_t>(d_num, stream, what);
}
}  // namespace detail

namespace detail {
// What a selection kernel tests.  A recognised predicate on arithmetic elements is evaluated
// inside the kernel on the elements themselves (or on the stencil); any other predicate is
// evaluated first, by a kernel instantiated for it, into one byte per element, and the
// selection kernel takes those bytes as its stencil.
template <typename St, typename Pred,
          bool InKernel = selects_in_kernel<Pred, typename std::remove_const<typename iterator_value<St>::type>::type>::value>
class tested_stream {
 public:
  typedef typename std::remove_const<typename iterator_value<St>::type>::type tested_type;
  typedef Pred predicate_type;
  tested_stream(void* stream, const temp_source& source, St tested, uint64_t n, Pred pred, bool has_stencil)
      : input_(stream, source, tested, has_stencil ? n : 0), pred_(pred), has_stencil_(has_stencil) {}
  const void* stencil() const { return has_stencil_ ? (const void*)input_.ptr() : nullptr; }
  int dtype() const { return dtype_of<tested_type>::value; }
  const Pred& predicate() const { return pred_; }

 private:
  device_input<St> input_;
  mutable Pred pred_;  // a caller's predicate need not be const-callable
  bool has_stencil_;
};
template <typename St, typename Pred>
class tested_stream<St, Pred, false> {
 public:
  typedef unsigned char tested_type;
  typedef thrust::identity<unsigned char> predicate_type;
  tested_stream(void* stream, const temp_source& source, St tested, uint64_t n, Pred pred, bool)
      : flags_(stream, source, thrust::make_transform_iterator(tested, as_flag<Pred>{pred}), n) {}
  const void* stencil() const { return flags_.ptr(); }
  int dtype() const { return THRUST_AMD_U8; }
  predicate_type predicate() const { return predicate_type(); }

 private:
  device_input<thrust::transform_iterator<as_flag<Pred>, St> > flags_;
};

#if defined(__HIPCC__)
// route 1: the predicate runs inside the compaction kernel
template <typename D, typename In, typename St, typename HasStencil, typename Out, typename Pred>
Out copy_if_impl(execution_policy<D>& exec, In first, In last, St stencil, HasStencil, Out result, Pred pred,
                 bool negate, std::integral_constant<int, 1>) {
  typedef typename std::remove_const<typename iterator_value<In>::type>::type T;
  typedef typename std::remove_const<typename iterator_value<St>::type>::type S;
  void* stream = stream_of(exec);
  const uint64_t n = (uint64_t)(last - first);
  if (n == 0) return result;
  device_input<In> source(stream, temp_source_of(exec), first, n);
  device_input<St> tested(stream, temp_source_of(exec), stencil, HasStencil::value ? n : 0);
  const uint64_t cnt = generic_selection<HasStencil::value>(
      stream, temp_source_of(exec), (const T*)source.ptr(), (const S*)tested.ptr(), thrust::detail::raw(result),
      (T*)nullptr, false, n, pred, negate, "copy_if failed");
  return result + cnt;
}
#endif
template <typename D, typename In, typename St, typename HasStencil, typename Out, typename Pred, int ROUTE>
Out copy_if_impl(execution_policy<D>& exec, In first, In last, St stencil, HasStencil, Out result, Pred pred,
                 bool negate, std::integral_constant<int, ROUTE>) {
  typedef typename std::remove_const<typename iterator_value<In>::type>::type T;
  const bool has_stencil = HasStencil::value;
  void* stream = stream_of(exec);
  const uint64_t n = (uint64_t)(last - first);
  if (n == 0) return result;
  device_input<In> source(stream, temp_source_of(exec), first, n);
  tested_stream<St, Pred> tested(stream, temp_source_of(exec), stencil, n, pred, has_stencil);
  const uint64_t cnt = run_selection<typename tested_stream<St, Pred>::tested_type>(
      stream, temp_source_of(exec), tested.predicate(), "copy_if failed",
      [&](void* t, std::size_t* b, uint64_t* d_num, int cmp, const void* thr) {
        return thrust_amd_copy_if(t, b, source.ptr(), tested.stencil(), thrust::detail::raw(result), d_num, n,
                                  sizeof(T), tested.dtype(), cmp, thr, stream);
      },
      negate);
  return result + cnt;
}
template <typename D, typename In, typename St, typename HasStencil, typename Out, typename Pred>
Out copy_if_impl(execution_policy<D>& exec, In first, In last, St stencil, HasStencil has_stencil, Out result,
                 Pred pred, bool negate) {
  typedef typename std::remove_const<typename iterator_value<St>::type>::type S;
  return copy_if_impl(exec, first, last, stencil, has_stencil, result, pred, negate, selection_route<Pred, S>());
}
}  // namespace detail

namespace detail {
// Items of 1, 2, 4 or 8 bytes into an array of the same type: the compaction kernels.  Anything
// else (wider elements, a zip or discard iterator as output, another output type): the
// three-pass selection through the iterators themselves.
template <typename D, typename In, typename St, typename HasStencil, typename Out, typename Pred>
Out copy_if_any(execution_policy<D>& exec, In first, In last, St stencil, HasStencil has_stencil, Out result, Pred pred,
                bool negate, std::true_type) {
  return copy_if_impl(exec, first, last, stencil, has_stencil, result, pred, negate);
}
template <typename D, typename In, typename St, typename HasStencil, typename Out, typename Pred>
Out copy_if_any(execution_policy<D>& exec, In first, In last, St stencil, HasStencil, Out result, Pred pred, bool negate,
                std::false_type) {
#if defined(__HIPCC__)
  const uint64_t n = (uint64_t)(last - first);
  return result + select_any_range<false>(exec, first, n, stencil, result, result, pred, negate, "copy_if failed");
#else
  static_assert(fancy_needs_hipcc<Pred>::value,
                "thrust::copy_if / remove_copy_if on the device system: items other than 1, 2, 4 or 8 bytes, and outputs "
                "that are not arrays of the input's type, are handled by kernels instantiated for the iterators; "
                "compile this translation unit with hipcc");
  return result;
#endif
}
template <typename D, typename In, typename St, typename HasStencil, typename Out, typename Pred>
Out copy_if_any(execution_policy<D>& exec, In first, In last, St stencil, HasStencil has_stencil, Out result, Pred pred,
                bool negate) {
  typedef typename std::remove_const<typename iterator_value<In>::type>::type T;
  return copy_if_any(exec, first, last, stencil, has_stencil, result, pred, negate,
                     std::integral_constant<bool, is_abi_item<T>::value && is_array_of<T, Out>::value>());
}
}  // namespace detail

template <typename D, typename In, typename Out, typename Pred>
Out copy_if(execution_policy<D>& exec, In first, In last, Out result, Pred pred) {
  return detail::copy_if_any(exec, first, last, first, std::false_type(), result, pred, false);
}
template <typename D, typename In, typename St, typename Out, typename Pred>
Out copy_if(execution_policy<D>& exec, In first, In last, St stencil, Out result, Pred pred) {
  return detail::copy_if_any(exec, first, last, stencil, std::true_type(), result, pred, false);
}
}  // namespace hip
}  // namespace system

// ------------------------------------------------------------------ copy
template <typename D, typename In, typename Out>
Out copy(const detail::execution_policy_base<D>& exec, In first, In last, Out result) {
  return copy(detail::derived_cast(detail::strip_const(exec)), first, last, result);
}
// Without a policy the two iterators may live in different systems.
namespace detail {
template <typename In, typename Out>
Out copy_any(In first, In last, Out result, std::false_type) {
  return copy_dispatch(first, last, result, is_device_iterator<In>::value, is_device_iterator<Out>::value, nullptr);
}
template <typename In, typename Out>
Out copy_any(In first, In last, Out result, std::true_type) {  // a fancy end: the output's system decides
  return thrust::copy(policy_for<Out>(), first, last, result);
}
}  // namespace detail
template <typename In, typename Out>
Out copy(In first, In last, Out result) {
  return detail::copy_any(first, last, result,
                          std::integral_constant<bool, detail::is_fancy_iterator<In>::value ||
                                                           detail::is_fancy_iterator<Out>::value>());
}
template <typename D, typename In, typename Size, typename Out>
Out copy_n(const detail::execution_policy_base<D>& exec, In first, Size n, Out result) {
  return thrust::copy(exec, first, first + n, result);
}
template <typename In, typename Size, typename Out,
          typename = typename std::enable_if<!detail::is_execution_policy<In>::value>::type>
Out copy_n(In first, Size n, Out result) {
  return thrust::copy(first, first + n, result);
}

// ------------------------------------------------------------------ copy_if
template <typename D, typename In, typename Out, typename Pred>
Out copy_if(const detail::execution_policy_base<D>& exec, In first, In last, Out result, Pred pred) {
  return copy_if(detail::derived_cast(detail::strip_const(exec)), first, last, result, pred);
}
template <typename D, typename In, typename St, typename Out, typename Pred>
Out copy_if(const detail::execution_policy_base<D>& exec, In first, In last, St stencil, Out result, Pred pred) {
  return copy_if(detail::derived_cast(detail::strip_const(exec)), first, last, stencil, result, pred);
}
template <typename In, typename Out, typename Pred>
Out copy_if(In first, In last, Out result, Pred pred) {
  return thrust::copy_if(detail::policy_for<In>(), first, last, result, pred);
}
template <typename In, typename St, typename Out, typename Pred,
          typename = typename std::enable_if<!detail::is_execution_policy<In>::value>::type>
Out copy_if(In first, In last, St stencil, Out result, Pred pred) {
  return thrust::copy_if(detail::policy_for<In>(), first, last, stencil, result, pred);
}

}  // namespace thrust
