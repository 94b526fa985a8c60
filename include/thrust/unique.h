// thrust::unique, unique_copy, unique_by_key, unique_by_key_copy.
//
// Keeps the first element of every run of consecutive equal elements
// (thrust/system/detail/generic/unique.inl:59-106, unique_by_key.inl:56-133).  The
// in-place forms run the copy form onto the input itself, which the device kernel
// supports (the reference's GPU path does the same, thrust/system/cuda/detail/unique.h:772).
#pragma once
#include <thrust/functional.h>
#include <thrust/pair.h>
#include <thrust/system/hip/detail/backend.h>
#include <thrust/system/hip/detail/device_input.h>
#include <thrust/system/hip/detail/staged_output.h>
#include <thrust/copy.h>
#if defined(__HIPCC__)
#include <thrust/system/hip/detail/generic_by_key.h>
#endif

namespace thrust {

template <typename D, typename In, typename Out, typename Pred>
Out unique_copy(const detail::execution_policy_base<D>& exec, In first, In last, Out result, Pred pred);
template <typename D, typename KIn, typename VIn, typename KOut, typename VOut, typename Pred>
pair<KOut, VOut> unique_by_key_copy(const detail::execution_policy_base<D>& exec, KIn kf, KIn kl, VIn vf,
                                    KOut ko, VOut vo, Pred pred);

namespace system {
namespace detail {
namespace generic {
template <typename D, typename It>
It unique(thrust::execution_policy<D>& exec, It first, It last) {
  typedef typename iterator_value<It>::type T;
  return thrust::unique_copy(exec, first, last, first, thrust::equal_to<T>());
}
template <typename D, typename It, typename Pred>
It unique(thrust::execution_policy<D>& exec, It first, It last, Pred pred) {
  return thrust::unique_copy(exec, first, last, first, pred);
}
template <typename D, typename In, typename Out>
Out unique_copy(thrust::execution_policy<D>& exec, In first, In last, Out result) {
  typedef typename iterator_value<In>::type T;
  return thrust::unique_copy(exec, first, last, result, thrust::equal_to<T>());
}
template <typename D, typename KIt, typename VIt>
pair<KIt, VIt> unique_by_key(thrust::execution_policy<D>& exec, KIt kf, KIt kl, VIt vf) {
  typedef typename iterator_value<KIt>::type K;
  return thrust::unique_by_key_copy(exec, kf, kl, vf, kf, vf, thrust::equal_to<K>());
}
template <typename D, typename KIt, typename VIt, typename Pred>
pair<KIt, VIt> unique_by_key(thrust::execution_policy<D>& exec, KIt kf, KIt kl, VIt vf, Pred pred) {
  return thrust::unique_by_key_copy(exec, kf, kl, vf, kf, vf, pred);
}
template <typename D, typename KIn, typename VIn, typename KOut, typename VOut>
pair<KOut, VOut> unique_by_key_copy(thrust::execution_policy<D>& exec, KIn kf, KIn kl, VIn vf, KOut ko, VOut vo) {
  typedef typename iterator_value<KIn>::type K;
  return thrust::unique_by_key_copy(exec, kf, kl, vf, ko, vo, thrust::equal_to<K>());
}
}  // namespace generic
}  // namespace detail

namespace cpp {
template <typename D, typename In, typename Out, typename Pred>
Out unique_copy(execution_policy<D>&, In first, In last, Out result, Pred pred) {
  typedef typename iterator_value<In>::type T;
  if (first == last) return result;
  T prev = *first;
  *result = prev; ++result;
  for (++first; first != last; ++first) {
    const T cur = *first;
    if (!pred(prev, cur)) { *result = cur; ++result; }
    prev = cur;
  }
  return result;
}
template <typename D, typename KIn, typename VIn, typename KOut, typename VOut, typename Pred>
pair<KOut, VOut> unique_by_key_copy(execution_policy<D>&, KIn kf, KIn kl, VIn vf, KOut ko, VOut vo, Pred pred) {
  typedef typename iterator_value<KIn>::type K;
  typedef typename iterator_value<VIn>::type V;
  if (kf == kl) return thrust::make_pair(ko, vo);
  K prev = *kf;
  { const V v = *vf; *ko = prev; ++ko; *vo = v; ++vo; }
  for (++kf, ++vf; kf != kl; ++kf, ++vf) {
    const K cur = *kf;
    const V v = *vf;
    if (!pred(prev, cur)) { *ko = cur; ++ko; *vo = v; ++vo; }
    prev = cur;
  }
  return thrust::make_pair(ko, vo);
}
}  // namespace cpp

namespace hip {
namespace detail {
template <typename K, typename KO, typename Pred, bool = is_abi_type<K>::value && std::is_same<KO, K>::value>
struct uniques_in_library : std::integral_constant<bool, is_equal_to<Pred, K>::value> {};
template <typename K, typename KO, typename Pred>
struct uniques_in_library<K, KO, Pred, false> : std::false_type {};

// a user's predicate or element struct: head flags from a kernel instantiated for it
template <typename D, typename In, typename Out, typename Pred>
Out unique_copy(execution_policy<D>& exec, In first, In last, Out result, Pred pred, std::false_type) {
#if defined(__HIPCC__)
  return unique_copy_generic(exec, first, last, result, pred);
#else
  static_assert(fancy_needs_hipcc<Pred>::value,
                "unique on the device system: predicates other than thrust::equal_to of an arithmetic type run in "
                "kernels instantiated for them; compile this translation unit with hipcc");
  return result;
#endif
}
template <typename D, typename KIn, typename VIn, typename KOut, typename VOut, typename Pred>
pair<KOut, VOut> unique_by_key_copy(execution_policy<D>& exec, KIn kf, KIn kl, VIn vf, KOut ko, VOut vo, Pred pred,
                                    std::false_type) {
#if defined(__HIPCC__)
  return unique_by_key_copy_generic(exec, kf, kl, vf, ko, vo, pred);
#else
  static_assert(fancy_needs_hipcc<Pred>::value,
                "unique_by_key on the device system: predicates other than thrust::equal_to of an arithmetic type run "
                "in kernels instantiated for them; compile this translation unit with hipcc");
  return thrust::make_pair(ko, vo);
#endif
}

template <typename D, typename In, typename Out, typename Pred>
Out unique_copy(execution_policy<D>& exec, In first, In last, Out result, Pred, std::true_type) {
  typedef typename std::remove_const<typename iterator_value<In>::type>::type T;
  void* stream = stream_of(exec);
  const uint64_t n = (uint64_t)(last - first);
  if (n == 0) return result;
  temp_storage temp(stream, temp_source_of(exec));
  uint64_t* d_num = nullptr;
  auto call = [&](void* t, std::size_t* b) {
    return thrust_amd_unique(t, b, thrust::detail::raw(first), thrust::detail::raw(result), d_num, n,
                             dtype_of<T>::value, stream);
  };
  std::size_t need = 0;
  throw_on_error(call(nullptr, &need), "unique: temp size query");
  const std::size_t aligned = (need + 255) / 256 * 256;
  temp.ensure(aligned + 256);
  d_num = reinterpret_cast<uint64_t*>(static_cast<char*>(temp.ptr()) + aligned);
  std::size_t bytes = aligned;
  throw_on_error(call(temp.ptr(), &bytes), "unique failed");
  return result + read_scalar<uint64_t>(d_num, stream, "unique: count copy");
}
template <typename D, typename KIn, typename VIn, typename KOut, typename VOut, typename Pred>
pair<KOut, VOut> unique_by_key_copy(execution_policy<D>& exec, KIn kf, KIn kl, VIn vf, KOut ko, VOut vo, Pred,
                                    std::true_type) {
  typedef typename std::remove_const<typename iterator_value<KIn>::type>::type K;
  typedef typename std::remove_const<typename iterator_value<VIn>::type>::type V;
  static_assert(is_abi_item<V>::value && std::is_same<typename iterator_value<VOut>::type, V>::value,
                "unique_by_key on the device system supports values of 1, 2, 4 or 8 bytes, same type in and out");
  void* stream = stream_of(exec);
  const uint64_t n = (uint64_t)(kl - kf);
  if (n == 0) return thrust::make_pair(ko, vo);
  temp_storage temp(stream, temp_source_of(exec));
  uint64_t* d_num = nullptr;
  auto call = [&](void* t, std::size_t* b) {
    return thrust_amd_unique_by_key(t, b, thrust::detail::raw(kf), thrust::detail::raw(vf), thrust::detail::raw(ko),
                                    thrust::detail::raw(vo), d_num, n, dtype_of<K>::value, sizeof(V), stream);
  };
  std::size_t need = 0;
  throw_on_error(call(nullptr, &need), "unique_by_key: temp size query");
  const std::size_t aligned = (need + 255) / 256 * 256;
  temp.ensure(aligned + 256);
  d_num = reinterpret_cast<uint64_t*>(static_cast<char*>(temp.ptr()) + aligned);
  std::size_t bytes = aligned;
  throw_on_error(call(temp.ptr(), &bytes), "unique_by_key failed");
  const uint64_t cnt = read_scalar<uint64_t>(d_num, stream, "unique_by_key: count copy");
  return thrust::make_pair(ko + cnt, vo + cnt);
}
}  // namespace detail

namespace detail {
template <typename D, typename In, typename Out, typename Pred>
Out unique_copy_staged(execution_policy<D>& exec, In first, In last, Out result, Pred pred, std::true_type) {
  typedef typename std::remove_const<typename iterator_value<In>::type>::type T;
  return unique_copy(exec, first, last, result, pred, uniques_in_library<T, typename iterator_value<Out>::type, Pred>());
}
template <typename D, typename KIn, typename VIn, typename KOut, typename VOut, typename Pred>
pair<KOut, VOut> unique_by_key_copy_staged(execution_policy<D>& exec, KIn kf, KIn kl, VIn vf, KOut ko, VOut vo,
                                           Pred pred, std::true_type) {
  typedef typename std::remove_const<typename iterator_value<KIn>::type>::type K;
  return unique_by_key_copy(exec, kf, kl, vf, ko, vo, pred,
                            uniques_in_library<K, typename iterator_value<KOut>::type, Pred>());
}
// an output that is not an array in memory: into temporary storage, then through the iterator
template <typename D, typename In, typename Out, typename Pred>
Out unique_copy_staged(execution_policy<D>& exec, In first, In last, Out result, Pred pred, std::false_type) {
  typedef typename std::remove_const<typename iterator_value<In>::type>::type T;
  output_stage<Out, T> out(stream_of(exec), temp_source_of(exec), result, (uint64_t)(last - first));
  const auto end = unique_copy_staged(exec, first, last, out.begin(), pred, std::true_type());
  return out.finish(exec, (uint64_t)(end - out.begin()));
}
template <typename D, typename KIn, typename VIn, typename KOut, typename VOut, typename Pred>
pair<KOut, VOut> unique_by_key_copy_staged(execution_policy<D>& exec, KIn kf, KIn kl, VIn vf, KOut ko, VOut vo,
                                           Pred pred, std::false_type) {
  typedef typename std::remove_const<typename iterator_value<KIn>::type>::type K;
  typedef typename std::remove_const<typename iterator_value<VIn>::type>::type V;
  const uint64_t n = (uint64_t)(kl - kf);
  output_stage<KOut, K> keys_out(stream_of(exec), temp_source_of(exec), ko, n);
  output_stage<VOut, V> values_out(stream_of(exec), temp_source_of(exec), vo, n);
  const auto ends = unique_by_key_copy_staged(exec, kf, kl, vf, keys_out.begin(), values_out.begin(), pred, std::true_type());
  const uint64_t runs = (uint64_t)(ends.first - keys_out.begin());
  return thrust::make_pair(keys_out.finish(exec, runs), values_out.finish(exec, runs));
}
}  // namespace detail

template <typename D, typename In, typename Out, typename Pred>
Out unique_copy(execution_policy<D>& exec, In first, In last, Out result, Pred pred) {
  return detail::unique_copy_staged(exec, first, last, result, pred,
                                    std::integral_constant<bool, detail::is_memory_iterator<Out>::value>());
}
template <typename D, typename KIn, typename VIn, typename KOut, typename VOut, typename Pred>
pair<KOut, VOut> unique_by_key_copy(execution_policy<D>& exec, KIn kf, KIn kl, VIn vf, KOut ko, VOut vo, Pred pred) {
  return detail::unique_by_key_copy_staged(
      exec, kf, kl, vf, ko, vo, pred,
      std::integral_constant<bool, detail::is_memory_iterator<KOut>::value && detail::is_memory_iterator<VOut>::value>());
}
}  // namespace hip
}  // namespace system

// ------------------------------------------------------------------ entry points
template <typename D, typename It>
It unique(const detail::execution_policy_base<D>& exec, It first, It last) {
  using thrust::system::detail::generic::unique;
  return unique(detail::derived_cast(detail::strip_const(exec)), first, last);
}
template <typename D, typename It, typename Pred>
It unique(const detail::execution_policy_base<D>& exec, It first, It last, Pred pred) {
  using thrust::system::detail::generic::unique;
  return unique(detail::derived_cast(detail::strip_const(exec)), first, last, pred);
}
template <typename It>
It unique(It first, It last) { return thrust::unique(detail::policy_for<It>(), first, last); }
template <typename It, typename Pred,
          typename = typename std::enable_if<!detail::is_execution_policy<It>::value>::type>
It unique(It first, It last, Pred pred) { return thrust::unique(detail::policy_for<It>(), first, last, pred); }

template <typename D, typename In, typename Out>
Out unique_copy(const detail::execution_policy_base<D>& exec, In first, In last, Out result) {
  using thrust::system::detail::generic::unique_copy;
  return unique_copy(detail::derived_cast(detail::strip_const(exec)), first, last, result);
}
template <typename D, typename In, typename Out, typename Pred>
Out unique_copy(const detail::execution_policy_base<D>& exec, In first, In last, Out result, Pred pred) {
  using thrust::system::detail::generic::unique_copy;
  return unique_copy(detail::derived_cast(detail::strip_const(exec)), first, last, result, pred);
}
template <typename In, typename Out>
Out unique_copy(In first, In last, Out result) {
  return thrust::unique_copy(detail::policy_for<In>(), first, last, result);
}
template <typename In, typename Out, typename Pred,
          typename = typename std::enable_if<!detail::is_execution_policy<In>::value>::type>
Out unique_copy(In first, In last, Out result, Pred pred) {
  return thrust::unique_copy(detail::policy_for<In>(), first, last, result, pred);
}

template <typename D, typename KIt, typename VIt>
pair<KIt, VIt> unique_by_key(const detail::execution_policy_base<D>& exec, KIt kf, KIt kl, VIt vf) {
  using thrust::system::detail::generic::unique_by_key;
  return unique_by_key(detail::derived_cast(detail::strip_const(exec)), kf, kl, vf);
}
template <typename D, typename KIt, typename VIt, typename Pred>
pair<KIt, VIt> unique_by_key(const detail::execution_policy_base<D>& exec, KIt kf, KIt kl, VIt vf, Pred pred) {
  using thrust::system::detail::generic::unique_by_key;
  return unique_by_key(detail::derived_cast(detail::strip_const(exec)), kf, kl, vf, pred);
}
template <typename KIt, typename VIt>
pair<KIt, VIt> unique_by_key(KIt kf, KIt kl, VIt vf) {
  return thrust::unique_by_key(detail::policy_for<KIt>(), kf, kl, vf);
}
template <typename KIt, typename VIt, typename Pred,
          typename = typename std::enable_if<!detail::is_execution_policy<KIt>::value>::type>
pair<KIt, VIt> unique_by_key(KIt kf, KIt kl, VIt vf, Pred pred) {
  return thrust::unique_by_key(detail::policy_for<KIt>(), kf, kl, vf, pred);
}

template <typename D, typename KIn, typename VIn, typename KOut, typename VOut>
pair<KOut, VOut> unique_by_key_copy(const detail::execution_policy_base<D>& exec, KIn kf, KIn kl, VIn vf,
                                    KOut ko, VOut vo) {
  using thrust::system::detail::generic::unique_by_key_copy;
  return unique_by_key_copy(detail::derived_cast(detail::strip_const(exec)), kf, kl, vf, ko, vo);
}
template <typename D, typename KIn, typename VIn, typename KOut, typename VOut, typename Pred>
pair<KOut, VOut> unique_by_key_copy(const detail::execution_policy_base<D>& exec, KIn kf, KIn kl, VIn vf,
                                    KOut ko, VOut vo, Pred pred) {
  using thrust::system::detail::generic::unique_by_key_copy;
  return unique_by_key_copy(detail::derived_cast(detail::strip_const(exec)), kf, kl, vf, ko, vo, pred);
}
template <typename KIn, typename VIn, typename KOut, typename VOut>
pair<KOut, VOut> unique_by_key_copy(KIn kf, KIn kl, VIn vf, KOut ko, VOut vo) {
  return thrust::unique_by_key_copy(detail::policy_for<KIn>(), kf, kl, vf, ko, vo);
}
template <typename KIn, typename VIn, typename KOut, typename VOut, typename Pred,
          typename = typename std::enable_if<!detail::is_execution_policy<KIn>::value>::type>
pair<KOut, VOut> unique_by_key_copy(KIn kf, KIn kl, VIn vf, KOut ko, VOut vo, Pred pred) {
  return thrust::unique_by_key_copy(detail::policy_for<KIn>(), kf, kl, vf, ko, vo, pred);
}

}  // namespace thrust
