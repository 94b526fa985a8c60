// thrust::sort, stable_sort, sort_by_key, stable_sort_by_key.
//
// As in the reference, sort is implemented as stable_sort on every system
// (thrust/system/detail/generic/sort.inl:57-64).  The device system takes the radix path
// for arithmetic keys with exactly thrust::less or thrust::greater -- the reference's own
// condition for its primitive sort (thrust/system/detail/sequential/sort.inl:139-148,
// thrust/system/cuda/detail/sort.h:1518-1523); other comparators are not available on
// the device system yet and fail to compile with a message.
#pragma once
#include <algorithm>
#include <numeric>
#include <vector>

#include <thrust/functional.h>
#include <thrust/system/hip/detail/backend.h>

namespace thrust {

template <typename D, typename It, typename Comp>
void stable_sort(const detail::execution_policy_base<D>& exec, It first, It last, Comp comp);
template <typename D, typename KIt, typename VIt, typename Comp>
void stable_sort_by_key(const detail::execution_policy_base<D>& exec, KIt keys_first, KIt keys_last,
                        VIt values_first, Comp comp);

namespace system {
namespace detail {
namespace generic {
template <typename D, typename It>
void sort(thrust::execution_policy<D>& exec, It first, It last) {
  typedef typename iterator_value<It>::type K;
  thrust::stable_sort(exec, first, last, thrust::less<K>());
}
template <typename D, typename It, typename Comp>
void sort(thrust::execution_policy<D>& exec, It first, It last, Comp comp) {
  thrust::stable_sort(exec, first, last, comp);
}
template <typename D, typename It>
void stable_sort(thrust::execution_policy<D>& exec, It first, It last) {
  typedef typename iterator_value<It>::type K;
  thrust::stable_sort(exec, first, last, thrust::less<K>());
}
template <typename D, typename KIt, typename VIt>
void sort_by_key(thrust::execution_policy<D>& exec, KIt kf, KIt kl, VIt vf) {
  typedef typename iterator_value<KIt>::type K;
  thrust::stable_sort_by_key(exec, kf, kl, vf, thrust::less<K>());
}
template <typename D, typename KIt, typename VIt, typename Comp>
void sort_by_key(thrust::execution_policy<D>& exec, KIt kf, KIt kl, VIt vf, Comp comp) {
  thrust::stable_sort_by_key(exec, kf, kl, vf, comp);
}
template <typename D, typename KIt, typename VIt>
void stable_sort_by_key(thrust::execution_policy<D>& exec, KIt kf, KIt kl, VIt vf) {
  typedef typename iterator_value<KIt>::type K;
  thrust::stable_sort_by_key(exec, kf, kl, vf, thrust::less<K>());
}
}  // namespace generic
}  // namespace detail

namespace cpp {
template <typename D, typename It, typename Comp>
void stable_sort(execution_policy<D>&, It first, It last, Comp comp) {
  std::stable_sort(first, last, comp);
}
template <typename D, typename KIt, typename VIt, typename Comp>
void stable_sort_by_key(execution_policy<D>&, KIt kf, KIt kl, VIt vf, Comp comp) {
  typedef typename iterator_value<KIt>::type K;
  typedef typename iterator_value<VIt>::type V;
  const std::size_t n = (std::size_t)(kl - kf);
  std::vector<std::size_t> order(n);
  std::iota(order.begin(), order.end(), std::size_t(0));
  std::stable_sort(order.begin(), order.end(), [&](std::size_t a, std::size_t b) { return comp(kf[a], kf[b]); });
  std::vector<K> k(n);
  std::vector<V> v(n);
  for (std::size_t i = 0; i < n; ++i) { k[i] = kf[order[i]]; v[i] = vf[order[i]]; }
  std::copy(k.begin(), k.end(), kf);
  std::copy(v.begin(), v.end(), vf);
}
}  // namespace cpp

namespace hip {
template <typename D, typename It, typename Comp>
void stable_sort(execution_policy<D>& exec, It first, It last, Comp) {
  typedef typename iterator_value<It>::type K;
  static_assert(std::is_pointer<It>::value || thrust::detail::is_device_iterator<It>::value,
                "sort on the device system needs device_ptr / device_vector iterators or raw device pointers");
  static_assert(detail::is_abi_type<K>::value && detail::order_code<Comp, K>::value >= 0,
                "sort on the device system supports arithmetic keys ordered by thrust::less or thrust::greater");
  void* stream = detail::stream_of(exec);
  const uint64_t n = (uint64_t)(last - first);
  if (n < 2) return;
  detail::temp_storage temp(stream, detail::temp_source_of(exec));
  detail::run(temp, 0, "sort failed", [&](void* t, std::size_t* b) {
    return thrust_amd_sort_keys(t, b, thrust::detail::raw(first), n, detail::dtype_of<K>::value,
                                detail::order_code<Comp, K>::value, 0, (int)sizeof(K) * 8, stream);
  });
  detail::synchronize(stream, "sort: synchronize");
}
template <typename D, typename KIt, typename VIt, typename Comp>
void stable_sort_by_key(execution_policy<D>& exec, KIt kf, KIt kl, VIt vf, Comp) {
  typedef typename iterator_value<KIt>::type K;
  typedef typename iterator_value<VIt>::type V;
  static_assert(detail::is_abi_type<K>::value && detail::order_code<Comp, K>::value >= 0,
                "sort_by_key on the device system supports arithmetic keys ordered by thrust::less or thrust::greater");
  static_assert(detail::is_abi_item<V>::value,
                "sort_by_key on the device system supports values of 1, 2, 4 or 8 bytes");
  void* stream = detail::stream_of(exec);
  const uint64_t n = (uint64_t)(kl - kf);
  if (n < 2) return;
  detail::temp_storage temp(stream, detail::temp_source_of(exec));
  detail::run(temp, 0, "sort_by_key failed", [&](void* t, std::size_t* b) {
    return thrust_amd_sort_pairs(t, b, thrust::detail::raw(kf), thrust::detail::raw(vf), n,
                                 detail::dtype_of<K>::value, sizeof(V), detail::order_code<Comp, K>::value, 0,
                                 (int)sizeof(K) * 8, stream);
  });
  detail::synchronize(stream, "sort_by_key: synchronize");
}
}  // namespace hip
}  // namespace system

#define THRUST_AMD_SORT_ENTRY(NAME)                                                                   \
  template <typename D, typename It>                                                                  \
  void NAME(const detail::execution_policy_base<D>& exec, It first, It last) {                        \
    using thrust::system::detail::generic::NAME;                                                      \
    NAME(detail::derived_cast(detail::strip_const(exec)), first, last);                               \
  }                                                                                                   \
  template <typename D, typename It, typename Comp>                                                   \
  void NAME(const detail::execution_policy_base<D>& exec, It first, It last, Comp comp) {             \
    using thrust::system::detail::generic::NAME;                                                      \
    NAME(detail::derived_cast(detail::strip_const(exec)), first, last, comp);                         \
  }                                                                                                   \
  template <typename It>                                                                              \
  void NAME(It first, It last) { thrust::NAME(detail::policy_for<It>(), first, last); }               \
  template <typename It, typename Comp,                                                               \
            typename = typename std::enable_if<!detail::is_execution_policy<It>::value>::type>        \
  void NAME(It first, It last, Comp comp) { thrust::NAME(detail::policy_for<It>(), first, last, comp); }
THRUST_AMD_SORT_ENTRY(sort)
THRUST_AMD_SORT_ENTRY(stable_sort)
#undef THRUST_AMD_SORT_ENTRY

#define THRUST_AMD_SORT_BY_KEY_ENTRY(NAME)                                                            \
  template <typename D, typename KIt, typename VIt>                                                   \
  void NAME(const detail::execution_policy_base<D>& exec, KIt kf, KIt kl, VIt vf) {                   \
    using thrust::system::detail::generic::NAME;                                                      \
    NAME(detail::derived_cast(detail::strip_const(exec)), kf, kl, vf);                                \
  }                                                                                                   \
  template <typename D, typename KIt, typename VIt, typename Comp>                                    \
  void NAME(const detail::execution_policy_base<D>& exec, KIt kf, KIt kl, VIt vf, Comp comp) {        \
    using thrust::system::detail::generic::NAME;                                                      \
    NAME(detail::derived_cast(detail::strip_const(exec)), kf, kl, vf, comp);                          \
  }                                                                                                   \
  template <typename KIt, typename VIt>                                                               \
  void NAME(KIt kf, KIt kl, VIt vf) { thrust::NAME(detail::policy_for<KIt>(), kf, kl, vf); }          \
  template <typename KIt, typename VIt, typename Comp,                                                \
            typename = typename std::enable_if<!detail::is_execution_policy<KIt>::value>::type>       \
  void NAME(KIt kf, KIt kl, VIt vf, Comp comp) { thrust::NAME(detail::policy_for<KIt>(), kf, kl, vf, comp); }
THRUST_AMD_SORT_BY_KEY_ENTRY(sort_by_key)
THRUST_AMD_SORT_BY_KEY_ENTRY(stable_sort_by_key)
#undef THRUST_AMD_SORT_BY_KEY_ENTRY

}  // namespace thrust
