// thrust::merge and thrust::merge_by_key.
//
// Stable merge of two sorted ranges; on ties the elements of the first range come first
// (thrust/system/detail/sequential/merge.inl:40-71,85-146).  The device system supports
// arithmetic keys ordered by thrust::less (default) or thrust::greater.
#pragma once
#include <thrust/functional.h>
#include <thrust/pair.h>
#include <thrust/system/hip/detail/backend.h>
#include <thrust/system/hip/detail/device_input.h>
#include <thrust/system/hip/detail/staged_output.h>
#include <thrust/copy.h>
#if defined(__HIPCC__)
#include <thrust/system/hip/detail/generic_select.h>
#include <thrust/system/hip/detail/merge_kernels.h>
#include <thrust/system/hip/detail/merge_sort_kernels.h>
#endif

namespace thrust {

template <typename D, typename In1, typename In2, typename Out, typename Comp>
Out merge(const detail::execution_policy_base<D>& exec, In1 first1, In1 last1, In2 first2, In2 last2, Out result,
          Comp comp);
template <typename D, typename K1, typename K2, typename V1, typename V2, typename KOut, typename VOut, typename Comp>
pair<KOut, VOut> merge_by_key(const detail::execution_policy_base<D>& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 vf1,
                              V2 vf2, KOut ko, VOut vo, Comp comp);

namespace system {
namespace detail {
namespace generic {
template <typename D, typename In1, typename In2, typename Out>
Out merge(thrust::execution_policy<D>& exec, In1 first1, In1 last1, In2 first2, In2 last2, Out result) {
  typedef typename iterator_value<In1>::type K;
  return thrust::merge(exec, first1, last1, first2, last2, result, thrust::less<K>());
}
template <typename D, typename K1, typename K2, typename V1, typename V2, typename KOut, typename VOut>
pair<KOut, VOut> merge_by_key(thrust::execution_policy<D>& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 vf1, V2 vf2,
                              KOut ko, VOut vo) {
  typedef typename iterator_value<K1>::type K;
  return thrust::merge_by_key(exec, kf1, kl1, kf2, kl2, vf1, vf2, ko, vo, thrust::less<K>());
}
}  // namespace generic
}  // namespace detail

namespace cpp {
template <typename D, typename In1, typename In2, typename Out, typename Comp>
Out merge(execution_policy<D>&, In1 first1, In1 last1, In2 first2, In2 last2, Out result, Comp comp) {
  while (first1 != last1 && first2 != last2) {
    if (comp(*first2, *first1)) { *result = *first2; ++first2; }
    else { *result = *first1; ++first1; }
    ++result;
  }
  for (; first1 != last1; ++first1, ++result) *result = *first1;
  for (; first2 != last2; ++first2, ++result) *result = *first2;
  return result;
}
template <typename D, typename K1, typename K2, typename V1, typename V2, typename KOut, typename VOut, typename Comp>
pair<KOut, VOut> merge_by_key(execution_policy<D>&, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 vf1, V2 vf2, KOut ko, VOut vo,
                              Comp comp) {
  while (kf1 != kl1 && kf2 != kl2) {
    if (comp(*kf2, *kf1)) { *ko = *kf2; *vo = *vf2; ++kf2; ++vf2; }
    else { *ko = *kf1; *vo = *vf1; ++kf1; ++vf1; }
    ++ko; ++vo;
  }
  for (; kf1 != kl1; ++kf1, ++vf1, ++ko, ++vo) { *ko = *kf1; *vo = *vf1; }
  for (; kf2 != kl2; ++kf2, ++vf2, ++ko, ++vo) { *ko = *kf2; *vo = *vf2; }
  return thrust::make_pair(ko, vo);
}
}  // namespace cpp

namespace hip {
namespace detail {
template <typename D, typename In1, typename In2, typename Out, typename Comp>
Out merge(execution_policy<D>& exec, In1 first1, In1 last1, In2 first2, In2 last2, Out result, Comp, std::true_type) {
  typedef typename std::remove_const<typename iterator_value<In1>::type>::type K;
  static_assert(is_abi_type<K>::value &&
                    std::is_same<typename std::remove_const<typename iterator_value<In2>::type>::type, K>::value &&
                    std::is_same<typename iterator_value<Out>::type, K>::value,
                "merge on the device system needs one arithmetic key type for both inputs and the output");
  static_assert(order_code<Comp, K>::value >= 0,
                "merge on the device system supports thrust::less and thrust::greater");
  void* stream = stream_of(exec);
  const uint64_t na = (uint64_t)(last1 - first1), nb = (uint64_t)(last2 - first2);
  if (na + nb == 0) return result;
  temp_storage temp(stream, temp_source_of(exec));
  run(temp, 0, "merge failed", [&](void* t, std::size_t* b) {
    return thrust_amd_merge(t, b, na ? thrust::detail::raw(first1) : nullptr, na,
                            nb ? thrust::detail::raw(first2) : nullptr, nb, thrust::detail::raw(result),
                            dtype_of<K>::value, order_code<Comp, K>::value, stream);
  });
  synchronize(stream, "merge: synchronize");
  return result + (na + nb);
}
template <typename D, typename K1, typename K2, typename V1, typename V2, typename KOut, typename VOut, typename Comp>
pair<KOut, VOut> merge_by_key(execution_policy<D>& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 vf1, V2 vf2, KOut ko,
                              VOut vo, Comp, std::true_type) {
  typedef typename std::remove_const<typename iterator_value<K1>::type>::type K;
  typedef typename std::remove_const<typename iterator_value<V1>::type>::type V;
  static_assert(is_abi_type<K>::value &&
                    std::is_same<typename std::remove_const<typename iterator_value<K2>::type>::type, K>::value &&
                    std::is_same<typename iterator_value<KOut>::type, K>::value,
                "merge_by_key on the device system needs one arithmetic key type for both inputs and the output");
  static_assert(is_abi_item<V>::value &&
                    std::is_same<typename std::remove_const<typename iterator_value<V2>::type>::type, V>::value &&
                    std::is_same<typename iterator_value<VOut>::type, V>::value,
                "merge_by_key on the device system supports values of 1, 2, 4 or 8 bytes, one type throughout");
  static_assert(order_code<Comp, K>::value >= 0,
                "merge_by_key on the device system supports thrust::less and thrust::greater");
  void* stream = stream_of(exec);
  const uint64_t na = (uint64_t)(kl1 - kf1), nb = (uint64_t)(kl2 - kf2);
  if (na + nb == 0) return thrust::make_pair(ko, vo);
  temp_storage temp(stream, temp_source_of(exec));
  run(temp, 0, "merge_by_key failed", [&](void* t, std::size_t* b) {
    return thrust_amd_merge_by_key(t, b, na ? thrust::detail::raw(kf1) : nullptr, na,
                                   nb ? thrust::detail::raw(kf2) : nullptr, nb,
                                   na ? thrust::detail::raw(vf1) : nullptr, nb ? thrust::detail::raw(vf2) : nullptr,
                                   thrust::detail::raw(ko), thrust::detail::raw(vo), dtype_of<K>::value,
                                   sizeof(V), order_code<Comp, K>::value, stream);
  });
  synchronize(stream, "merge_by_key: synchronize");
  return thrust::make_pair(ko + (na + nb), vo + (na + nb));
}

// A user's comparator or key type: both ranges are written one behind the other into temporary
// storage (which also reads fancy iterators) and merged by the merge sort's kernels.
template <typename D, typename K1, typename K2, typename V1, typename V2, typename KOut, typename VOut, typename Comp>
void merge_generic(execution_policy<D>& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 vf1, V2 vf2, KOut ko, VOut vo,
                   Comp comp, bool has_values) {
#if defined(__HIPCC__)
  namespace ms = thrust::system::hip::merge_sort;
  typedef typename std::remove_const<typename iterator_value<K1>::type>::type K;
  typedef typename iterator_value<VOut>::type V;
  static_assert(std::is_same<typename iterator_value<KOut>::type, K>::value,
                "merge on the device system: the output holds the first range's key type");
  void* stream = stream_of(exec);
  const uint64_t na = (uint64_t)(kl1 - kf1), nb = (uint64_t)(kl2 - kf2), n = na + nb;
  if (n == 0) return;
  // keys (and values) of up to 8 bytes: the merge-path kernels of the library, instantiated for
  // the comparator, read the two ranges where they lie (fancy iterators are written out first)
  if constexpr (is_kernel_item<K>::value && sizeof(K) <= 8 && is_kernel_item<V>::value && sizeof(V) <= 8 &&
                std::is_same<typename std::remove_const<typename iterator_value<K2>::type>::type, K>::value) {
    namespace mg = thrust::system::hip::merging;
    device_input<K1> a(stream, temp_source_of(exec), kf1, na);
    device_input<K2> b(stream, temp_source_of(exec), kf2, nb);
    temp_storage temp(stream, temp_source_of(exec));
    temp.ensure(mg::merge_temp_bytes(n));
    int rc;
    if (has_values) {
      typedef typename std::remove_const<typename iterator_value<V1>::type>::type Va;
      typedef typename std::remove_const<typename iterator_value<V2>::type>::type Vb;
      static_assert(std::is_same<Va, Vb>::value, "merge_by_key on the device system: one value type for both ranges");
      device_input<V1> va(stream, temp_source_of(exec), vf1, na);
      device_input<V2> vb(stream, temp_source_of(exec), vf2, nb);
      rc = mg::merge_launch<K, Va, true>(static_cast<uint64_t*>(temp.ptr()), (const K*)a.ptr(), na, (const K*)b.ptr(), nb,
                                         (const Va*)va.ptr(), (const Va*)vb.ptr(), thrust::detail::raw(ko),
                                         (Va*)thrust::detail::raw(vo), comp, (hipStream_t)stream);
    } else {
      rc = mg::merge_launch<K, uint32_t, false>(static_cast<uint64_t*>(temp.ptr()), (const K*)a.ptr(), na,
                                                (const K*)b.ptr(), nb, (const uint32_t*)nullptr, (const uint32_t*)nullptr,
                                                thrust::detail::raw(ko), (uint32_t*)nullptr, comp, (hipStream_t)stream);
    }
    throw_on_error(rc, "merge failed");
    synchronize(stream, "merge: synchronize");
    return;
  }
  const uint64_t tiles = (n + ms::TILE - 1) / ms::TILE;
  const std::size_t key_bytes = ((std::size_t)n * sizeof(K) + 255) / 256 * 256;
  const std::size_t val_bytes = has_values ? ((std::size_t)n * sizeof(V) + 255) / 256 * 256 : 0;
  temp_storage temp(stream, temp_source_of(exec));
  temp.ensure(key_bytes + val_bytes + (std::size_t)(tiles + 1) * sizeof(uint64_t));
  K* both = static_cast<K*>(temp.ptr());
  V* both_values = reinterpret_cast<V*>(static_cast<char*>(temp.ptr()) + key_bytes);
  uint64_t* split = reinterpret_cast<uint64_t*>(static_cast<char*>(temp.ptr()) + key_bytes + val_bytes);
  materialize(stream, kf1, both, na);
  materialize(stream, kf2, both + na, nb);
  int rc;
  if (has_values) {
    materialize(stream, vf1, both_values, na);
    materialize(stream, vf2, both_values + na, nb);
    rc = ms::merge_two<K, V, true>(both, both_values, na, n, thrust::detail::raw(ko), thrust::detail::raw(vo), split,
                                   comp, (hipStream_t)stream);
  } else {
    rc = ms::merge_two<K, V, false>(both, (const V*)nullptr, na, n, thrust::detail::raw(ko), (V*)nullptr, split, comp,
                                    (hipStream_t)stream);
  }
  throw_on_error(rc, "merge failed");
  synchronize(stream, "merge: synchronize");
#else
  static_assert(fancy_needs_hipcc<Comp>::value,
                "merge on the device system: comparators other than thrust::less / thrust::greater of an arithmetic key "
                "run in kernels instantiated for the comparator; compile this translation unit with hipcc");
#endif
}
template <typename D, typename In1, typename In2, typename Out, typename Comp>
Out merge(execution_policy<D>& exec, In1 first1, In1 last1, In2 first2, In2 last2, Out result, Comp comp, std::false_type) {
  merge_generic(exec, first1, last1, first2, last2, first1, first2, result, result, comp, false);
  return result + ((last1 - first1) + (last2 - first2));
}
template <typename D, typename K1, typename K2, typename V1, typename V2, typename KOut, typename VOut, typename Comp>
pair<KOut, VOut> merge_by_key(execution_policy<D>& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 vf1, V2 vf2, KOut ko,
                              VOut vo, Comp comp, std::false_type) {
  merge_generic(exec, kf1, kl1, kf2, kl2, vf1, vf2, ko, vo, comp, true);
  const std::ptrdiff_t n = (kl1 - kf1) + (kl2 - kf2);
  return thrust::make_pair(ko + n, vo + n);
}

template <typename K, typename K2, typename KO, typename Comp,
          bool = is_abi_type<K>::value && std::is_same<K2, K>::value && std::is_same<KO, K>::value>
struct merges_in_library : std::integral_constant<bool, (order_code<Comp, K>::value >= 0)> {};
template <typename K, typename K2, typename KO, typename Comp>
struct merges_in_library<K, K2, KO, Comp, false> : std::false_type {};
}  // namespace detail

namespace detail {
template <typename D, typename In1, typename In2, typename Out, typename Comp>
Out merge_staged(execution_policy<D>& exec, In1 first1, In1 last1, In2 first2, In2 last2, Out result, Comp comp,
                 std::true_type) {
  typedef typename std::remove_const<typename iterator_value<In1>::type>::type K;
  typedef typename std::remove_const<typename iterator_value<In2>::type>::type K2;
  return merge(exec, first1, last1, first2, last2, result, comp,
               merges_in_library<K, K2, typename iterator_value<Out>::type, Comp>());
}
template <typename D, typename K1, typename K2, typename V1, typename V2, typename KOut, typename VOut, typename Comp>
pair<KOut, VOut> merge_by_key_staged(execution_policy<D>& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 vf1, V2 vf2, KOut ko,
                                     VOut vo, Comp comp, std::true_type) {
  typedef typename std::remove_const<typename iterator_value<K1>::type>::type K;
  typedef typename std::remove_const<typename iterator_value<K2>::type>::type Kb;
  return merge_by_key(exec, kf1, kl1, kf2, kl2, vf1, vf2, ko, vo, comp,
                      merges_in_library<K, Kb, typename iterator_value<KOut>::type, Comp>());
}
// an output that is not an array in memory (discard_iterator, a zip): into temporary storage,
// then through the iterator
template <typename D, typename In1, typename In2, typename Out, typename Comp>
Out merge_staged(execution_policy<D>& exec, In1 first1, In1 last1, In2 first2, In2 last2, Out result, Comp comp,
                 std::false_type) {
  typedef typename std::remove_const<typename iterator_value<In1>::type>::type K;
  const uint64_t n = (uint64_t)(last1 - first1) + (uint64_t)(last2 - first2);
  output_stage<Out, K> out(stream_of(exec), temp_source_of(exec), result, n);
  merge_staged(exec, first1, last1, first2, last2, out.begin(), comp, std::true_type());
  return out.finish(exec, n);
}
template <typename D, typename K1, typename K2, typename V1, typename V2, typename KOut, typename VOut, typename Comp>
pair<KOut, VOut> merge_by_key_staged(execution_policy<D>& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 vf1, V2 vf2, KOut ko,
                                     VOut vo, Comp comp, std::false_type) {
  typedef typename std::remove_const<typename iterator_value<K1>::type>::type K;
  typedef typename std::remove_const<typename iterator_value<V1>::type>::type V;
  const uint64_t n = (uint64_t)(kl1 - kf1) + (uint64_t)(kl2 - kf2);
  output_stage<KOut, K> keys_out(stream_of(exec), temp_source_of(exec), ko, n);
  output_stage<VOut, V> values_out(stream_of(exec), temp_source_of(exec), vo, n);
  merge_by_key_staged(exec, kf1, kl1, kf2, kl2, vf1, vf2, keys_out.begin(), values_out.begin(), comp, std::true_type());
  return thrust::make_pair(keys_out.finish(exec, n), values_out.finish(exec, n));
}
}  // namespace detail

template <typename D, typename In1, typename In2, typename Out, typename Comp>
Out merge(execution_policy<D>& exec, In1 first1, In1 last1, In2 first2, In2 last2, Out result, Comp comp) {
  return detail::merge_staged(exec, first1, last1, first2, last2, result, comp,
                              std::integral_constant<bool, detail::is_memory_iterator<Out>::value>());
}
template <typename D, typename K1, typename K2, typename V1, typename V2, typename KOut, typename VOut, typename Comp>
pair<KOut, VOut> merge_by_key(execution_policy<D>& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 vf1, V2 vf2, KOut ko,
                              VOut vo, Comp comp) {
  return detail::merge_by_key_staged(
      exec, kf1, kl1, kf2, kl2, vf1, vf2, ko, vo, comp,
      std::integral_constant<bool, detail::is_memory_iterator<KOut>::value && detail::is_memory_iterator<VOut>::value>());
}
}  // namespace hip
}  // namespace system

// ------------------------------------------------------------------ entry points
template <typename D, typename In1, typename In2, typename Out>
Out merge(const detail::execution_policy_base<D>& exec, In1 first1, In1 last1, In2 first2, In2 last2, Out result) {
  using thrust::system::detail::generic::merge;
  return merge(detail::derived_cast(detail::strip_const(exec)), first1, last1, first2, last2, result);
}
template <typename D, typename In1, typename In2, typename Out, typename Comp>
Out merge(const detail::execution_policy_base<D>& exec, In1 first1, In1 last1, In2 first2, In2 last2, Out result,
          Comp comp) {
  using thrust::system::detail::generic::merge;
  return merge(detail::derived_cast(detail::strip_const(exec)), first1, last1, first2, last2, result, comp);
}
template <typename In1, typename In2, typename Out>
Out merge(In1 first1, In1 last1, In2 first2, In2 last2, Out result) {
  return thrust::merge(detail::policy_for<In1>(), first1, last1, first2, last2, result);
}
template <typename In1, typename In2, typename Out, typename Comp,
          typename = typename std::enable_if<!detail::is_execution_policy<In1>::value>::type>
Out merge(In1 first1, In1 last1, In2 first2, In2 last2, Out result, Comp comp) {
  return thrust::merge(detail::policy_for<In1>(), first1, last1, first2, last2, result, comp);
}

template <typename D, typename K1, typename K2, typename V1, typename V2, typename KOut, typename VOut>
pair<KOut, VOut> merge_by_key(const detail::execution_policy_base<D>& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 vf1,
                              V2 vf2, KOut ko, VOut vo) {
  using thrust::system::detail::generic::merge_by_key;
  return merge_by_key(detail::derived_cast(detail::strip_const(exec)), kf1, kl1, kf2, kl2, vf1, vf2, ko, vo);
}
template <typename D, typename K1, typename K2, typename V1, typename V2, typename KOut, typename VOut, typename Comp>
pair<KOut, VOut> merge_by_key(const detail::execution_policy_base<D>& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 vf1,
                              V2 vf2, KOut ko, VOut vo, Comp comp) {
  using thrust::system::detail::generic::merge_by_key;
  return merge_by_key(detail::derived_cast(detail::strip_const(exec)), kf1, kl1, kf2, kl2, vf1, vf2, ko, vo, comp);
}
template <typename K1, typename K2, typename V1, typename V2, typename KOut, typename VOut>
pair<KOut, VOut> merge_by_key(K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 vf1, V2 vf2, KOut ko, VOut vo) {
  return thrust::merge_by_key(detail::policy_for<K1>(), kf1, kl1, kf2, kl2, vf1, vf2, ko, vo);
}
template <typename K1, typename K2, typename V1, typename V2, typename KOut, typename VOut, typename Comp,
          typename = typename std::enable_if<!detail::is_execution_policy<K1>::value>::type>
pair<KOut, VOut> merge_by_key(K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 vf1, V2 vf2, KOut ko, VOut vo, Comp comp) {
  return thrust::merge_by_key(detail::policy_for<K1>(), kf1, kl1, kf2, kl2, vf1, vf2, ko, vo, comp);
}

}  // namespace thrust
