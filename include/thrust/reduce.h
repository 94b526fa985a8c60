// thrust::reduce and thrust::reduce_by_key.
//
// Overload set as in the reference (thrust/detail/reduce.inl:34-72,141-187 and
// :75-138,190-274): with and without an execution policy; reduce(first,last) uses
// init = value_type(0) and plus<value_type>, i.e. an integer sum wraps in the value type
// (thrust/system/detail/generic/reduce.inl:35-53).
#pragma once
#include <thrust/functional.h>
#include <thrust/pair.h>
#include <thrust/system/hip/detail/backend.h>
#include <thrust/system/hip/detail/device_input.h>
#include <thrust/system/hip/detail/staged_output.h>
#include <thrust/copy.h>
#if defined(__HIPCC__)
#include <thrust/system/hip/detail/generic_kernels.h>
#include <thrust/system/hip/detail/generic_by_key.h>
#endif

namespace thrust {

// ------------------------------------------------------------------ entry points
template <typename D, typename It>
typename iterator_value<It>::type reduce(const detail::execution_policy_base<D>& exec, It first, It last);
template <typename D, typename It, typename T>
T reduce(const detail::execution_policy_base<D>& exec, It first, It last, T init);
template <typename D, typename It, typename T, typename Op>
T reduce(const detail::execution_policy_base<D>& exec, It first, It last, T init, Op op);

template <typename D, typename KIt, typename VIt, typename KOut, typename VOut>
pair<KOut, VOut> reduce_by_key(const detail::execution_policy_base<D>& exec, KIt keys_first, KIt keys_last,
                               VIt values_first, KOut keys_output, VOut values_output);
template <typename D, typename KIt, typename VIt, typename KOut, typename VOut, typename Pred>
pair<KOut, VOut> reduce_by_key(const detail::execution_policy_base<D>& exec, KIt keys_first, KIt keys_last,
                               VIt values_first, KOut keys_output, VOut values_output, Pred pred);
template <typename D, typename KIt, typename VIt, typename KOut, typename VOut, typename Pred, typename Op>
pair<KOut, VOut> reduce_by_key(const detail::execution_policy_base<D>& exec, KIt keys_first, KIt keys_last,
                               VIt values_first, KOut keys_output, VOut values_output, Pred pred, Op op);

namespace system {
namespace detail {
namespace generic {
// Defaulting chain (thrust/system/detail/generic/reduce.inl:35-53, reduce_by_key.inl:139-190).
template <typename D, typename It>
typename iterator_value<It>::type reduce(thrust::execution_policy<D>& exec, It first, It last) {
  typedef typename iterator_value<It>::type T;
  return thrust::reduce(exec, first, last, T(0));
}
template <typename D, typename It, typename T>
T reduce(thrust::execution_policy<D>& exec, It first, It last, T init) {
  return thrust::reduce(exec, first, last, init, thrust::plus<T>());
}
template <typename D, typename KIt, typename VIt, typename KOut, typename VOut>
pair<KOut, VOut> reduce_by_key(thrust::execution_policy<D>& exec, KIt kf, KIt kl, VIt vf, KOut ko, VOut vo) {
  typedef typename iterator_value<KIt>::type K;
  return thrust::reduce_by_key(exec, kf, kl, vf, ko, vo, thrust::equal_to<K>());
}
template <typename D, typename KIt, typename VIt, typename KOut, typename VOut, typename Pred>
pair<KOut, VOut> reduce_by_key(thrust::execution_policy<D>& exec, KIt kf, KIt kl, VIt vf, KOut ko, VOut vo,
                               Pred pred) {
  typedef typename iterator_value<VIt>::type V;
  return thrust::reduce_by_key(exec, kf, kl, vf, ko, vo, pred, thrust::plus<V>());
}
}  // namespace generic
}  // namespace detail

namespace cpp {
// Sequential host system (thrust/system/detail/sequential/reduce.h:39-66, reduce_by_key.h:36-98).
template <typename D, typename It, typename T, typename Op>
T reduce(execution_policy<D>&, It first, It last, T init, Op op) {
  for (; first != last; ++first) init = op(init, *first);
  return init;
}
template <typename D, typename KIt, typename VIt, typename KOut, typename VOut, typename Pred, typename Op>
pair<KOut, VOut> reduce_by_key(execution_policy<D>&, KIt kf, KIt kl, VIt vf, KOut ko, VOut vo, Pred pred, Op op) {
  typedef typename iterator_value<KIt>::type K;
  typedef typename iterator_value<VIt>::type V;
  if (kf == kl) return thrust::make_pair(ko, vo);
  K run_key = *kf;
  V acc = *vf;
  for (++kf, ++vf; kf != kl; ++kf, ++vf) {
    const K k = *kf;
    if (pred(run_key, k)) {  // against the key that opened the run, not the previous one
      acc = op(acc, *vf);
    } else {
      *ko = run_key; ++ko;
      *vo = acc; ++vo;
      run_key = k;
      acc = *vf;
    }
  }
  *ko = run_key; ++ko;
  *vo = acc; ++vo;
  return thrust::make_pair(ko, vo);
}
}  // namespace cpp

namespace hip {
// The accumulator has the type of init; elements of another arithmetic type are converted
// to it first, as plus<T> does in the reference (testing/reduce.cu:99-129).
namespace detail {
template <typename D, typename It, typename T, typename Op>
T reduce(execution_policy<D>& exec, It first, It last, T init, Op, std::true_type) {
  void* stream = stream_of(exec);
  const uint64_t n = (uint64_t)(last - first);
  device_input<It> source(stream, temp_source_of(exec), first, n);
  temp_storage converted(stream, temp_source_of(exec));
  const void* in = n ? (const void*)input_as<T>(source.ptr(), n, stream, converted) : nullptr;
  temp_storage temp(stream, temp_source_of(exec));
  void* d_out = nullptr;
  // the result slot is the `extra` region, which run() only knows after the size query
  std::size_t need = 0;
  throw_on_error(thrust_amd_reduce(nullptr, &need, in, n, dtype_of<T>::value,
                                           binop_code<Op, T>::value, &init, nullptr, stream),
                         "reduce: temp size query");
  const std::size_t aligned = (need + 255) / 256 * 256;
  temp.ensure(aligned + 256);
  d_out = static_cast<char*>(temp.ptr()) + aligned;
  std::size_t bytes = aligned;
  throw_on_error(thrust_amd_reduce(temp.ptr(), &bytes, in, n, dtype_of<T>::value,
                                           binop_code<Op, T>::value, &init, d_out, stream),
                         "reduce failed");
  return read_scalar<T>(d_out, stream, "reduce: result copy");
}

// A user's operator or element type: kernels instantiated for them (hipcc translation units).
template <typename D, typename It, typename T, typename Op>
T reduce(execution_policy<D>& exec, It first, It last, T init, Op op, std::false_type) {
#if defined(__HIPCC__)
  namespace gk = thrust::system::hip::generic;
  typedef typename thrust::detail::device_view_of<It>::type View;
  void* stream = stream_of(exec);
  const uint64_t n = (uint64_t)(last - first);
  if (n == 0) return init;
  uint64_t chunks = (n + gk::TILE - 1) / gk::TILE;
  if (chunks > 1024) chunks = 1024;
  const uint64_t chunk = (n + chunks - 1) / chunks;
  chunks = (n + chunk - 1) / chunk;  // every chunk holds at least one element
  const std::size_t partial_bytes = ((std::size_t)chunks * sizeof(T) + 255) / 256 * 256;
  temp_storage temp(stream, temp_source_of(exec));
  temp.ensure(partial_bytes + 256);
  T* partials = static_cast<T*>(temp.ptr());
  T* d_out = reinterpret_cast<T*>(static_cast<char*>(temp.ptr()) + partial_bytes);
  hipLaunchKernelGGL((gk::reduce_chunks_kernel<View, T, Op>), dim3((unsigned)chunks), dim3(gk::BLOCK), 0,
                     (hipStream_t)stream, thrust::detail::device_view(first), n, chunk, op, partials);
  throw_on_error(launch_status(), "reduce: kernel launch");
  hipLaunchKernelGGL((gk::reduce_final_kernel<T, Op>), dim3(1), dim3(gk::BLOCK), 0, (hipStream_t)stream,
                     (const T*)partials, (uint32_t)chunks, init, op, d_out);
  throw_on_error(launch_status(), "reduce: kernel launch");
  return read_scalar<T>(d_out, stream, "reduce: result copy");
#else
  static_assert(fancy_needs_hipcc<Op>::value,
                "thrust::reduce on the device system: fancy iterators, and operators other than thrust::plus / minimum / "
                "maximum of an arithmetic type, run in kernels instantiated for them; compile this translation unit with hipcc");
  return init;
#endif
}

template <typename T, typename V, typename Op, bool = is_abi_type<T>::value && is_abi_type<V>::value>
struct reduces_in_library : std::integral_constant<bool, (binop_code<Op, T>::value >= 0)> {};
template <typename T, typename V, typename Op>
struct reduces_in_library<T, V, Op, false> : std::false_type {};
}  // namespace detail

template <typename D, typename It, typename T, typename Op>
T reduce(execution_policy<D>& exec, It first, It last, T init, Op op) {
  typedef typename std::remove_const<typename iterator_value<It>::type>::type V;
  static_assert(detail::is_device_input<It>::value,
                "thrust::reduce on the device system needs device_ptr / device_vector iterators, raw device pointers "
                "or fancy iterators over them");
  // a fancy iterator is read where it is (the kernels instantiated for it), not written out first
  return detail::reduce(exec, first, last, init, op,
                        std::integral_constant<bool, detail::reduces_in_library<T, V, Op>::value &&
                                                         !thrust::detail::is_fancy_iterator<It>::value>());
}

namespace detail {
// library path: arithmetic keys and values, equal_to, plus / minimum / maximum, same types in and out
template <typename K, typename V, typename KO, typename VO, typename Pred, typename Op,
          bool = is_abi_type<K>::value && is_abi_type<V>::value && std::is_same<KO, K>::value && std::is_same<VO, V>::value>
struct reduces_by_key_in_library
    : std::integral_constant<bool, is_equal_to<Pred, K>::value && (binop_code<Op, V>::value >= 0)> {};
template <typename K, typename V, typename KO, typename VO, typename Pred, typename Op>
struct reduces_by_key_in_library<K, V, KO, VO, Pred, Op, false> : std::false_type {};

template <typename D, typename KIt, typename VIt, typename KOut, typename VOut, typename Pred, typename Op>
pair<KOut, VOut> reduce_by_key(execution_policy<D>& exec, KIt kf, KIt kl, VIt vf, KOut ko, VOut vo, Pred pred, Op op,
                               std::false_type) {
#if defined(__HIPCC__)
  return reduce_by_key_generic(exec, kf, kl, vf, ko, vo, pred, op);
#else
  static_assert(fancy_needs_hipcc<Op>::value,
                "thrust::reduce_by_key on the device system: key predicates other than thrust::equal_to, operators other "
                "than thrust::plus / minimum / maximum and non-arithmetic elements run in kernels instantiated for "
                "them; compile this translation unit with hipcc");
  return thrust::make_pair(ko, vo);
#endif
}
template <typename D, typename KIt, typename VIt, typename KOut, typename VOut, typename Pred, typename Op>
pair<KOut, VOut> reduce_by_key(execution_policy<D>& exec, KIt kf, KIt kl, VIt vf, KOut ko, VOut vo, Pred, Op,
                               std::true_type) {
  typedef typename std::remove_const<typename iterator_value<KIt>::type>::type K;
  typedef typename std::remove_const<typename iterator_value<VIt>::type>::type V;
  void* stream = stream_of(exec);
  const uint64_t n = (uint64_t)(kl - kf);
  if (n == 0) return thrust::make_pair(ko, vo);
  device_input<KIt> keys_in(stream, temp_source_of(exec), kf, n);
  device_input<VIt> values_in(stream, temp_source_of(exec), vf, n);
  temp_storage temp(stream, temp_source_of(exec));
  uint64_t* d_runs = nullptr;
  std::size_t need = 0;
  auto call = [&](void* t, std::size_t* b) {
    return thrust_amd_reduce_by_key(t, b, keys_in.ptr(), values_in.ptr(),
                                    thrust::detail::raw(ko), thrust::detail::raw(vo), d_runs, n,
                                    dtype_of<K>::value, dtype_of<V>::value,
                                    binop_code<Op, V>::value, stream);
  };
  throw_on_error(call(nullptr, &need), "reduce_by_key: temp size query");
  const std::size_t aligned = (need + 255) / 256 * 256;
  temp.ensure(aligned + 256);
  d_runs = reinterpret_cast<uint64_t*>(static_cast<char*>(temp.ptr()) + aligned);
  std::size_t bytes = aligned;
  throw_on_error(call(temp.ptr(), &bytes), "reduce_by_key failed");
  const uint64_t runs = read_scalar<uint64_t>(d_runs, stream, "reduce_by_key: count copy");
  return thrust::make_pair(ko + runs, vo + runs);
}
}  // namespace detail

namespace detail {
template <typename D, typename KIt, typename VIt, typename KOut, typename VOut, typename Pred, typename Op>
pair<KOut, VOut> reduce_by_key_staged(execution_policy<D>& exec, KIt kf, KIt kl, VIt vf, KOut ko, VOut vo, Pred pred,
                                      Op op, std::true_type) {
  typedef typename std::remove_const<typename iterator_value<KIt>::type>::type K;
  typedef typename std::remove_const<typename iterator_value<VIt>::type>::type V;
  return reduce_by_key(exec, kf, kl, vf, ko, vo, pred, op,
                       reduces_by_key_in_library<K, V, typename iterator_value<KOut>::type,
                                                 typename iterator_value<VOut>::type, Pred, Op>());
}
// an output that is not an array in memory: into temporary storage, then through the iterator
template <typename D, typename KIt, typename VIt, typename KOut, typename VOut, typename Pred, typename Op>
pair<KOut, VOut> reduce_by_key_staged(execution_policy<D>& exec, KIt kf, KIt kl, VIt vf, KOut ko, VOut vo, Pred pred,
                                      Op op, std::false_type) {
  typedef typename std::remove_const<typename iterator_value<KIt>::type>::type K;
  typedef typename std::remove_const<typename iterator_value<VIt>::type>::type V;
  const uint64_t n = (uint64_t)(kl - kf);
  output_stage<KOut, K> keys_out(stream_of(exec), temp_source_of(exec), ko, n);
  output_stage<VOut, V> sums_out(stream_of(exec), temp_source_of(exec), vo, n);
  const auto ends = reduce_by_key_staged(exec, kf, kl, vf, keys_out.begin(), sums_out.begin(), pred, op, std::true_type());
  const uint64_t runs = (uint64_t)(ends.first - keys_out.begin());
  return thrust::make_pair(keys_out.finish(exec, runs), sums_out.finish(exec, runs));
}
}  // namespace detail

template <typename D, typename KIt, typename VIt, typename KOut, typename VOut, typename Pred, typename Op>
pair<KOut, VOut> reduce_by_key(execution_policy<D>& exec, KIt kf, KIt kl, VIt vf, KOut ko, VOut vo, Pred pred, Op op) {
  return detail::reduce_by_key_staged(
      exec, kf, kl, vf, ko, vo, pred, op,
      std::integral_constant<bool, detail::is_memory_iterator<KOut>::value && detail::is_memory_iterator<VOut>::value>());
}
}  // namespace hip
}  // namespace system

// ------------------------------------------------------------------ entry point bodies
template <typename D, typename It>
typename iterator_value<It>::type reduce(const detail::execution_policy_base<D>& exec, It first, It last) {
  using thrust::system::detail::generic::reduce;
  return reduce(detail::derived_cast(detail::strip_const(exec)), first, last);
}
template <typename D, typename It, typename T>
T reduce(const detail::execution_policy_base<D>& exec, It first, It last, T init) {
  using thrust::system::detail::generic::reduce;
  return reduce(detail::derived_cast(detail::strip_const(exec)), first, last, init);
}
template <typename D, typename It, typename T, typename Op>
T reduce(const detail::execution_policy_base<D>& exec, It first, It last, T init, Op op) {
  using thrust::system::detail::generic::reduce;
  return reduce(detail::derived_cast(detail::strip_const(exec)), first, last, init, op);
}
template <typename It>
typename iterator_value<It>::type reduce(It first, It last) {
  return thrust::reduce(detail::policy_for<It>(), first, last);
}
template <typename It, typename T>
T reduce(It first, It last, T init) {
  return thrust::reduce(detail::policy_for<It>(), first, last, init);
}
template <typename It, typename T, typename Op>
T reduce(It first, It last, T init, Op op) {
  return thrust::reduce(detail::policy_for<It>(), first, last, init, op);
}

template <typename D, typename KIt, typename VIt, typename KOut, typename VOut>
pair<KOut, VOut> reduce_by_key(const detail::execution_policy_base<D>& exec, KIt kf, KIt kl, VIt vf, KOut ko,
                               VOut vo) {
  using thrust::system::detail::generic::reduce_by_key;
  return reduce_by_key(detail::derived_cast(detail::strip_const(exec)), kf, kl, vf, ko, vo);
}
template <typename D, typename KIt, typename VIt, typename KOut, typename VOut, typename Pred>
pair<KOut, VOut> reduce_by_key(const detail::execution_policy_base<D>& exec, KIt kf, KIt kl, VIt vf, KOut ko,
                               VOut vo, Pred pred) {
  using thrust::system::detail::generic::reduce_by_key;
  return reduce_by_key(detail::derived_cast(detail::strip_const(exec)), kf, kl, vf, ko, vo, pred);
}
template <typename D, typename KIt, typename VIt, typename KOut, typename VOut, typename Pred, typename Op>
pair<KOut, VOut> reduce_by_key(const detail::execution_policy_base<D>& exec, KIt kf, KIt kl, VIt vf, KOut ko,
                               VOut vo, Pred pred, Op op) {
  using thrust::system::detail::generic::reduce_by_key;
  return reduce_by_key(detail::derived_cast(detail::strip_const(exec)), kf, kl, vf, ko, vo, pred, op);
}
template <typename KIt, typename VIt, typename KOut, typename VOut>
pair<KOut, VOut> reduce_by_key(KIt kf, KIt kl, VIt vf, KOut ko, VOut vo) {
  return thrust::reduce_by_key(detail::policy_for<KIt>(), kf, kl, vf, ko, vo);
}
template <typename KIt, typename VIt, typename KOut, typename VOut, typename Pred,
          typename = typename std::enable_if<!detail::is_execution_policy<KIt>::value>::type>
pair<KOut, VOut> reduce_by_key(KIt kf, KIt kl, VIt vf, KOut ko, VOut vo, Pred pred) {
  return thrust::reduce_by_key(detail::policy_for<KIt>(), kf, kl, vf, ko, vo, pred);
}
template <typename KIt, typename VIt, typename KOut, typename VOut, typename Pred, typename Op,
          typename = typename std::enable_if<!detail::is_execution_policy<KIt>::value>::type>
pair<KOut, VOut> reduce_by_key(KIt kf, KIt kl, VIt vf, KOut ko, VOut vo, Pred pred, Op op) {
  return thrust::reduce_by_key(detail::policy_for<KIt>(), kf, kl, vf, ko, vo, pred, op);
}

}  // namespace thrust
