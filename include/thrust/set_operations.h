// thrust::set_difference, set_intersection, set_symmetric_difference, set_union and their
// _by_key forms.
//
// Both inputs are sorted by comp (default thrust::less); equal keys are multisets: a key
// with m copies in the first range and n in the second appears max(m-n,0), min(m,n),
// |m-n| or max(m,n) times, and the copies that survive are those the reference's
// sequential loops keep (thrust/system/detail/sequential/set_operations.h:42-215): the
// first range's first min(m,n) copies for intersection, its last m-n for difference, and
// for union all of the first range followed by the second range's last n-m.  The _by_key
// forms carry one value with every kept key, taken from the range the key came from
// (thrust/system/detail/generic/set_operations.inl:44-330).  On the device system,
// arithmetic keys ordered by thrust::less or thrust::greater run in the library's kernels;
// other comparators and key structs run in kernels instantiated for them, in translation
// units compiled with hipcc.  Results must not overlap the inputs.
#pragma once
#include <thrust/functional.h>
#include <thrust/pair.h>
#include <thrust/system/hip/detail/backend.h>
#include <thrust/system/hip/detail/device_input.h>
#include <thrust/system/hip/detail/staged_output.h>
#include <thrust/copy.h>
#if defined(__HIPCC__)
#include <thrust/system/hip/detail/generic_set_operations.h>
#endif

namespace thrust {
namespace system {

namespace cpp {
namespace detail {
// The two-pointer loop shared by the four operations; OP is a thrust_amd_set_op code.
// `emit1(i)` / `emit2(j)` output the current element of the first / second range.
template <int OP, typename K1, typename K2, typename Comp, typename Emit1, typename Emit2>
inline void set_operation_loop(K1 f1, K1 l1, K2 f2, K2 l2, Comp comp, Emit1 emit1, Emit2 emit2) {
  const bool both_tails = OP == THRUST_AMD_SET_SYMMETRIC_DIFFERENCE || OP == THRUST_AMD_SET_UNION;
  while (f1 != l1 && f2 != l2) {
    if (comp(*f1, *f2)) {
      if (OP != THRUST_AMD_SET_INTERSECTION) emit1(f1);
      ++f1;
    } else if (comp(*f2, *f1)) {
      if (both_tails) emit2(f2);
      ++f2;
    } else {
      if (OP == THRUST_AMD_SET_INTERSECTION || OP == THRUST_AMD_SET_UNION) emit1(f1);
      ++f1;
      ++f2;
    }
  }
  if (OP != THRUST_AMD_SET_INTERSECTION)
    for (; f1 != l1; ++f1) emit1(f1);
  if (both_tails)
    for (; f2 != l2; ++f2) emit2(f2);
}
template <int OP, typename In1, typename In2, typename Out, typename Comp>
inline Out set_operation(In1 f1, In1 l1, In2 f2, In2 l2, Out result, Comp comp) {
  set_operation_loop<OP>(f1, l1, f2, l2, comp, [&](In1 p) { *result = *p; ++result; },
                         [&](In2 p) { *result = *p; ++result; });
  return result;
}
// vf2 may be a null placeholder (intersection never reads it)
template <int OP, typename K1, typename K2, typename V1, typename V2, typename KOut, typename VOut, typename Comp>
inline pair<KOut, VOut> set_operation_by_key(K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 vf1, V2 vf2, KOut ko, VOut vo,
                                             Comp comp) {
  const K1 k1_begin = kf1;
  const K2 k2_begin = kf2;
  set_operation_loop<OP>(kf1, kl1, kf2, kl2, comp,
                         [&](K1 p) { *ko = *p; *vo = *(vf1 + (p - k1_begin)); ++ko; ++vo; },
                         [&](K2 p) { *ko = *p; *vo = *(vf2 + (p - k2_begin)); ++ko; ++vo; });
  return thrust::make_pair(ko, vo);
}
}  // namespace detail
}  // namespace cpp

namespace hip {
namespace detail {
// The library's kernels take one arithmetic key type throughout, ordered by operator< or operator>.
template <typename K, typename In2, typename Out, typename Comp,
          bool = is_abi_type<K>::value &&
                 std::is_same<typename std::remove_const<typename iterator_value<In2>::type>::type, K>::value &&
                 std::is_same<typename iterator_value<Out>::type, K>::value>
struct set_operation_in_library : std::integral_constant<bool, (order_code<Comp, K>::value >= 0)> {};
template <typename K, typename In2, typename Out, typename Comp>
struct set_operation_in_library<K, In2, Out, Comp, false> : std::false_type {};

// Everything else: kernels instantiated for the comparator.
template <int OP, typename D, typename K1, typename K2, typename V1, typename V2, typename KOut, typename VOut,
          typename Comp>
inline uint64_t set_operation_other(execution_policy<D>& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 vf1, V2 vf2, KOut ko,
                                    VOut vo, Comp comp, bool has_values) {
#if defined(__HIPCC__)
  return set_operation_generic<OP>(exec, kf1, kl1, kf2, kl2, vf1, vf2, ko, vo, comp, has_values);
#else
  static_assert(fancy_needs_hipcc<Comp>::value,
                "set operations on the device system: comparators other than thrust::less / thrust::greater of an "
                "arithmetic key run in kernels instantiated for the comparator; compile this translation unit with hipcc");
  return 0;
#endif
}

template <int OP, typename D, typename In1, typename In2, typename Out, typename Comp>
inline Out set_operation(execution_policy<D>& exec, In1 first1, In1 last1, In2 first2, In2 last2, Out result, Comp comp,
                         std::false_type) {
  return result + set_operation_other<OP>(exec, first1, last1, first2, last2, first1, first2, result, result, comp, false);
}

template <int OP, typename D, typename In1, typename In2, typename Out, typename Comp>
inline Out set_operation(execution_policy<D>& exec, In1 first1, In1 last1, In2 first2, In2 last2, Out result, Comp,
                         std::true_type) {
  typedef typename std::remove_const<typename iterator_value<In1>::type>::type K;
  void* stream = stream_of(exec);
  const uint64_t na = (uint64_t)(last1 - first1), nb = (uint64_t)(last2 - first2);
  if (na + nb == 0) return result;
  temp_storage temp(stream, temp_source_of(exec));
  uint64_t* d_num = nullptr;
  std::size_t need = 0;
  auto call = [&](void* t, std::size_t* b) {
    return thrust_amd_set_operation(t, b, OP, na ? thrust::detail::raw(first1) : nullptr, na,
                                    nb ? thrust::detail::raw(first2) : nullptr, nb, thrust::detail::raw(result), d_num,
                                    dtype_of<K>::value, order_code<Comp, K>::value, stream);
  };
  throw_on_error(call(nullptr, &need), "set operation: temp size query");
  const std::size_t aligned = (need + 255) / 256 * 256;
  temp.ensure(aligned + 256);
  d_num = reinterpret_cast<uint64_t*>(static_cast<char*>(temp.ptr()) + aligned);
  std::size_t bytes = aligned;
  throw_on_error(call(temp.ptr(), &bytes), "set operation failed");
  return result + read_scalar<uint64_t>(d_num, stream, "set operation: result size");
}

template <int OP, typename D, typename In1, typename In2, typename Out, typename Comp>
inline Out set_operation_staged(execution_policy<D>& exec, In1 first1, In1 last1, In2 first2, In2 last2, Out result,
                                Comp comp, std::true_type) {
  typedef typename std::remove_const<typename iterator_value<In1>::type>::type K;
  return set_operation<OP>(exec, first1, last1, first2, last2, result, comp,
                           set_operation_in_library<K, In2, Out, Comp>());
}
// an output that is not an array in memory (discard_iterator, a zip): into temporary storage,
// then through the iterator
template <int OP, typename D, typename In1, typename In2, typename Out, typename Comp>
inline Out set_operation_staged(execution_policy<D>& exec, In1 first1, In1 last1, In2 first2, In2 last2, Out result,
                                Comp comp, std::false_type) {
  typedef typename std::remove_const<typename iterator_value<In1>::type>::type K;
  const uint64_t capacity = (uint64_t)(last1 - first1) + (uint64_t)(last2 - first2);
  output_stage<Out, K> out(stream_of(exec), temp_source_of(exec), result, capacity);
  const auto end = set_operation_staged<OP>(exec, first1, last1, first2, last2, out.begin(), comp, std::true_type());
  return out.finish(exec, (uint64_t)(end - out.begin()));
}
template <int OP, typename D, typename In1, typename In2, typename Out, typename Comp>
inline Out set_operation(execution_policy<D>& exec, In1 first1, In1 last1, In2 first2, In2 last2, Out result, Comp comp) {
  return set_operation_staged<OP>(exec, first1, last1, first2, last2, result, comp,
                                  std::integral_constant<bool, is_memory_iterator<Out>::value>());
}

template <int OP, typename D, typename K1, typename K2, typename V1, typename V2, typename KOut, typename VOut,
          typename Comp>
inline pair<KOut, VOut> set_operation_by_key(execution_policy<D>& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 vf1, V2 vf2,
                                             KOut ko, VOut vo, Comp comp, std::false_type) {
  const uint64_t cnt = set_operation_other<OP>(exec, kf1, kl1, kf2, kl2, vf1, vf2, ko, vo, comp, true);
  return thrust::make_pair(ko + cnt, vo + cnt);
}

template <int OP, typename D, typename K1, typename K2, typename V1, typename V2, typename KOut, typename VOut,
          typename Comp>
inline pair<KOut, VOut> set_operation_by_key(execution_policy<D>& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 vf1, V2 vf2,
                                             KOut ko, VOut vo, Comp, std::true_type) {
  typedef typename std::remove_const<typename iterator_value<K1>::type>::type K;
  typedef typename std::remove_const<typename iterator_value<V1>::type>::type V;
  static_assert(is_abi_item<V>::value &&
                    std::is_same<typename std::remove_const<typename iterator_value<V2>::type>::type, V>::value &&
                    std::is_same<typename iterator_value<VOut>::type, V>::value,
                "set operations by key on the device system support values of 1, 2, 4 or 8 bytes, one type throughout");
  void* stream = stream_of(exec);
  const uint64_t na = (uint64_t)(kl1 - kf1), nb = (uint64_t)(kl2 - kf2);
  if (na + nb == 0) return thrust::make_pair(ko, vo);
  const bool keeps_second = OP == THRUST_AMD_SET_SYMMETRIC_DIFFERENCE || OP == THRUST_AMD_SET_UNION;
  temp_storage temp(stream, temp_source_of(exec));
  uint64_t* d_num = nullptr;
  std::size_t need = 0;
  auto call = [&](void* t, std::size_t* b) {
    return thrust_amd_set_operation_by_key(
        t, b, OP, na ? thrust::detail::raw(kf1) : nullptr, na, nb ? thrust::detail::raw(kf2) : nullptr, nb,
        na ? thrust::detail::raw(vf1) : nullptr, (nb && keeps_second) ? thrust::detail::raw(vf2) : nullptr,
        thrust::detail::raw(ko), thrust::detail::raw(vo), d_num, dtype_of<K>::value, sizeof(V),
        order_code<Comp, K>::value, stream);
  };
  throw_on_error(call(nullptr, &need), "set operation by key: temp size query");
  const std::size_t aligned = (need + 255) / 256 * 256;
  temp.ensure(aligned + 256);
  d_num = reinterpret_cast<uint64_t*>(static_cast<char*>(temp.ptr()) + aligned);
  std::size_t bytes = aligned;
  throw_on_error(call(temp.ptr(), &bytes), "set operation by key failed");
  const uint64_t cnt = read_scalar<uint64_t>(d_num, stream, "set operation by key: result size");
  return thrust::make_pair(ko + cnt, vo + cnt);
}

template <int OP, typename D, typename K1, typename K2, typename V1, typename V2, typename KOut, typename VOut,
          typename Comp>
inline pair<KOut, VOut> set_operation_by_key_staged(execution_policy<D>& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 vf1,
                                                    V2 vf2, KOut ko, VOut vo, Comp comp, std::true_type) {
  typedef typename std::remove_const<typename iterator_value<K1>::type>::type K;
  return set_operation_by_key<OP>(exec, kf1, kl1, kf2, kl2, vf1, vf2, ko, vo, comp,
                                  set_operation_in_library<K, K2, KOut, Comp>());
}
template <int OP, typename D, typename K1, typename K2, typename V1, typename V2, typename KOut, typename VOut,
          typename Comp>
inline pair<KOut, VOut> set_operation_by_key_staged(execution_policy<D>& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 vf1,
                                                    V2 vf2, KOut ko, VOut vo, Comp comp, std::false_type) {
  typedef typename std::remove_const<typename iterator_value<K1>::type>::type K;
  typedef typename std::remove_const<typename iterator_value<V1>::type>::type V;
  const uint64_t capacity = (uint64_t)(kl1 - kf1) + (uint64_t)(kl2 - kf2);
  output_stage<KOut, K> keys_out(stream_of(exec), temp_source_of(exec), ko, capacity);
  output_stage<VOut, V> values_out(stream_of(exec), temp_source_of(exec), vo, capacity);
  const auto ends = set_operation_by_key_staged<OP>(exec, kf1, kl1, kf2, kl2, vf1, vf2, keys_out.begin(),
                                                    values_out.begin(), comp, std::true_type());
  const uint64_t count = (uint64_t)(ends.first - keys_out.begin());
  return thrust::make_pair(keys_out.finish(exec, count), values_out.finish(exec, count));
}
template <int OP, typename D, typename K1, typename K2, typename V1, typename V2, typename KOut, typename VOut,
          typename Comp>
inline pair<KOut, VOut> set_operation_by_key(execution_policy<D>& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 vf1, V2 vf2,
                                             KOut ko, VOut vo, Comp comp) {
  return set_operation_by_key_staged<OP>(
      exec, kf1, kl1, kf2, kl2, vf1, vf2, ko, vo, comp,
      std::integral_constant<bool, is_memory_iterator<KOut>::value && is_memory_iterator<VOut>::value>());
}
}  // namespace detail
}  // namespace hip
}  // namespace system

// One operation on keys: declaration, defaulted comparison, the two systems, entry points.
#define THRUST_AMD_SET_OPERATION(NAME, OP)                                                                          \
  template <typename D, typename In1, typename In2, typename Out, typename Comp>                                    \
  Out NAME(const detail::execution_policy_base<D>& exec, In1 first1, In1 last1, In2 first2, In2 last2, Out result,  \
           Comp comp);                                                                                              \
  namespace system {                                                                                                \
  namespace detail {                                                                                                \
  namespace generic {                                                                                               \
  template <typename D, typename In1, typename In2, typename Out>                                                   \
  Out NAME(thrust::execution_policy<D>& exec, In1 first1, In1 last1, In2 first2, In2 last2, Out result) {           \
    typedef typename iterator_value<In1>::type K;                                                                   \
    return thrust::NAME(exec, first1, last1, first2, last2, result, thrust::less<K>());                             \
  }                                                                                                                 \
  }                                                                                                                 \
  }                                                                                                                 \
  namespace cpp {                                                                                                   \
  template <typename D, typename In1, typename In2, typename Out, typename Comp>                                    \
  Out NAME(execution_policy<D>&, In1 first1, In1 last1, In2 first2, In2 last2, Out result, Comp comp) {             \
    return detail::set_operation<OP>(first1, last1, first2, last2, result, comp);                                   \
  }                                                                                                                 \
  }                                                                                                                 \
  namespace hip {                                                                                                   \
  template <typename D, typename In1, typename In2, typename Out, typename Comp>                                    \
  Out NAME(execution_policy<D>& exec, In1 first1, In1 last1, In2 first2, In2 last2, Out result, Comp comp) {        \
    return detail::set_operation<OP>(exec, first1, last1, first2, last2, result, comp);                             \
  }                                                                                                                 \
  }                                                                                                                 \
  }                                                                                                                 \
  template <typename D, typename In1, typename In2, typename Out>                                                   \
  Out NAME(const detail::execution_policy_base<D>& exec, In1 first1, In1 last1, In2 first2, In2 last2, Out result) { \
    using thrust::system::detail::generic::NAME;                                                                    \
    return NAME(detail::derived_cast(detail::strip_const(exec)), first1, last1, first2, last2, result);             \
  }                                                                                                                 \
  template <typename D, typename In1, typename In2, typename Out, typename Comp>                                    \
  Out NAME(const detail::execution_policy_base<D>& exec, In1 first1, In1 last1, In2 first2, In2 last2, Out result,  \
           Comp comp) {                                                                                             \
    using thrust::system::detail::generic::NAME;                                                                    \
    return NAME(detail::derived_cast(detail::strip_const(exec)), first1, last1, first2, last2, result, comp);       \
  }                                                                                                                 \
  template <typename In1, typename In2, typename Out>                                                               \
  Out NAME(In1 first1, In1 last1, In2 first2, In2 last2, Out result) {                                              \
    return thrust::NAME(detail::policy_for<In1>(), first1, last1, first2, last2, result);                           \
  }                                                                                                                 \
  template <typename In1, typename In2, typename Out, typename Comp,                                                \
            typename = typename std::enable_if<!detail::is_execution_policy<In1>::value>::type>                     \
  Out NAME(In1 first1, In1 last1, In2 first2, In2 last2, Out result, Comp comp) {                                   \
    return thrust::NAME(detail::policy_for<In1>(), first1, last1, first2, last2, result, comp);                     \
  }

THRUST_AMD_SET_OPERATION(set_difference, THRUST_AMD_SET_DIFFERENCE)
THRUST_AMD_SET_OPERATION(set_intersection, THRUST_AMD_SET_INTERSECTION)
THRUST_AMD_SET_OPERATION(set_symmetric_difference, THRUST_AMD_SET_SYMMETRIC_DIFFERENCE)
THRUST_AMD_SET_OPERATION(set_union, THRUST_AMD_SET_UNION)
#undef THRUST_AMD_SET_OPERATION

// The by-key forms that take the values of both ranges.
#define THRUST_AMD_SET_OPERATION_BY_KEY(NAME, OP)                                                                   \
  template <typename D, typename K1, typename K2, typename V1, typename V2, typename KOut, typename VOut,           \
            typename Comp>                                                                                          \
  pair<KOut, VOut> NAME(const detail::execution_policy_base<D>& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 vf1,       \
                        V2 vf2, KOut ko, VOut vo, Comp comp);                                                       \
  namespace system {                                                                                                \
  namespace detail {                                                                                                \
  namespace generic {                                                                                               \
  template <typename D, typename K1, typename K2, typename V1, typename V2, typename KOut, typename VOut>           \
  pair<KOut, VOut> NAME(thrust::execution_policy<D>& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 vf1, V2 vf2, KOut ko, \
                        VOut vo) {                                                                                  \
    typedef typename iterator_value<K1>::type K;                                                                    \
    return thrust::NAME(exec, kf1, kl1, kf2, kl2, vf1, vf2, ko, vo, thrust::less<K>());                             \
  }                                                                                                                 \
  }                                                                                                                 \
  }                                                                                                                 \
  namespace cpp {                                                                                                   \
  template <typename D, typename K1, typename K2, typename V1, typename V2, typename KOut, typename VOut,           \
            typename Comp>                                                                                          \
  pair<KOut, VOut> NAME(execution_policy<D>&, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 vf1, V2 vf2, KOut ko, VOut vo,     \
                        Comp comp) {                                                                                \
    return detail::set_operation_by_key<OP>(kf1, kl1, kf2, kl2, vf1, vf2, ko, vo, comp);                            \
  }                                                                                                                 \
  }                                                                                                                 \
  namespace hip {                                                                                                   \
  template <typename D, typename K1, typename K2, typename V1, typename V2, typename KOut, typename VOut,           \
            typename Comp>                                                                                          \
  pair<KOut, VOut> NAME(execution_policy<D>& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 vf1, V2 vf2, KOut ko,         \
                        VOut vo, Comp comp) {                                                                       \
    return detail::set_operation_by_key<OP>(exec, kf1, kl1, kf2, kl2, vf1, vf2, ko, vo, comp);                      \
  }                                                                                                                 \
  }                                                                                                                 \
  }                                                                                                                 \
  template <typename D, typename K1, typename K2, typename V1, typename V2, typename KOut, typename VOut>           \
  pair<KOut, VOut> NAME(const detail::execution_policy_base<D>& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 vf1,       \
                        V2 vf2, KOut ko, VOut vo) {                                                                 \
    using thrust::system::detail::generic::NAME;                                                                    \
    return NAME(detail::derived_cast(detail::strip_const(exec)), kf1, kl1, kf2, kl2, vf1, vf2, ko, vo);             \
  }                                                                                                                 \
  template <typename D, typename K1, typename K2, typename V1, typename V2, typename KOut, typename VOut,           \
            typename Comp>                                                                                          \
  pair<KOut, VOut> NAME(const detail::execution_policy_base<D>& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 vf1,       \
                        V2 vf2, KOut ko, VOut vo, Comp comp) {                                                      \
    using thrust::system::detail::generic::NAME;                                                                    \
    return NAME(detail::derived_cast(detail::strip_const(exec)), kf1, kl1, kf2, kl2, vf1, vf2, ko, vo, comp);       \
  }                                                                                                                 \
  template <typename K1, typename K2, typename V1, typename V2, typename KOut, typename VOut>                       \
  pair<KOut, VOut> NAME(K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 vf1, V2 vf2, KOut ko, VOut vo) {                         \
    return thrust::NAME(detail::policy_for<K1>(), kf1, kl1, kf2, kl2, vf1, vf2, ko, vo);                            \
  }                                                                                                                 \
  template <typename K1, typename K2, typename V1, typename V2, typename KOut, typename VOut, typename Comp,        \
            typename = typename std::enable_if<!detail::is_execution_policy<K1>::value>::type>                      \
  pair<KOut, VOut> NAME(K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 vf1, V2 vf2, KOut ko, VOut vo, Comp comp) {              \
    return thrust::NAME(detail::policy_for<K1>(), kf1, kl1, kf2, kl2, vf1, vf2, ko, vo, comp);                      \
  }

THRUST_AMD_SET_OPERATION_BY_KEY(set_difference_by_key, THRUST_AMD_SET_DIFFERENCE)
THRUST_AMD_SET_OPERATION_BY_KEY(set_symmetric_difference_by_key, THRUST_AMD_SET_SYMMETRIC_DIFFERENCE)
THRUST_AMD_SET_OPERATION_BY_KEY(set_union_by_key, THRUST_AMD_SET_UNION)
#undef THRUST_AMD_SET_OPERATION_BY_KEY

// set_intersection_by_key takes the values of the first range only.
template <typename D, typename K1, typename K2, typename V1, typename KOut, typename VOut, typename Comp>
pair<KOut, VOut> set_intersection_by_key(const detail::execution_policy_base<D>& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2,
                                         V1 vf1, KOut ko, VOut vo, Comp comp);
namespace system {
namespace detail {
namespace generic {
template <typename D, typename K1, typename K2, typename V1, typename KOut, typename VOut>
pair<KOut, VOut> set_intersection_by_key(thrust::execution_policy<D>& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 vf1,
                                         KOut ko, VOut vo) {
  typedef typename iterator_value<K1>::type K;
  return thrust::set_intersection_by_key(exec, kf1, kl1, kf2, kl2, vf1, ko, vo, thrust::less<K>());
}
}  // namespace generic
}  // namespace detail
namespace cpp {
template <typename D, typename K1, typename K2, typename V1, typename KOut, typename VOut, typename Comp>
pair<KOut, VOut> set_intersection_by_key(execution_policy<D>&, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 vf1, KOut ko, VOut vo,
                                         Comp comp) {
  return detail::set_operation_by_key<THRUST_AMD_SET_INTERSECTION>(kf1, kl1, kf2, kl2, vf1, vf1, ko, vo, comp);
}
}  // namespace cpp
namespace hip {
template <typename D, typename K1, typename K2, typename V1, typename KOut, typename VOut, typename Comp>
pair<KOut, VOut> set_intersection_by_key(execution_policy<D>& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 vf1, KOut ko,
                                         VOut vo, Comp comp) {
  return detail::set_operation_by_key<THRUST_AMD_SET_INTERSECTION>(exec, kf1, kl1, kf2, kl2, vf1, vf1, ko, vo, comp);
}
}  // namespace hip
}  // namespace system
template <typename D, typename K1, typename K2, typename V1, typename KOut, typename VOut>
pair<KOut, VOut> set_intersection_by_key(const detail::execution_policy_base<D>& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2,
                                         V1 vf1, KOut ko, VOut vo) {
  using thrust::system::detail::generic::set_intersection_by_key;
  return set_intersection_by_key(detail::derived_cast(detail::strip_const(exec)), kf1, kl1, kf2, kl2, vf1, ko, vo);
}
template <typename D, typename K1, typename K2, typename V1, typename KOut, typename VOut, typename Comp>
pair<KOut, VOut> set_intersection_by_key(const detail::execution_policy_base<D>& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2,
                                         V1 vf1, KOut ko, VOut vo, Comp comp) {
  using thrust::system::detail::generic::set_intersection_by_key;
  return set_intersection_by_key(detail::derived_cast(detail::strip_const(exec)), kf1, kl1, kf2, kl2, vf1, ko, vo, comp);
}
template <typename K1, typename K2, typename V1, typename KOut, typename VOut>
pair<KOut, VOut> set_intersection_by_key(K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 vf1, KOut ko, VOut vo) {
  return thrust::set_intersection_by_key(detail::policy_for<K1>(), kf1, kl1, kf2, kl2, vf1, ko, vo);
}
template <typename K1, typename K2, typename V1, typename KOut, typename VOut, typename Comp,
          typename = typename std::enable_if<!detail::is_execution_policy<K1>::value>::type>
pair<KOut, VOut> set_intersection_by_key(K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 vf1, KOut ko, VOut vo, Comp comp) {
  return thrust::set_intersection_by_key(detail::policy_for<K1>(), kf1, kl1, kf2, kl2, vf1, ko, vo, comp);
}

}  // namespace thrust
