// thrust::sort, stable_sort, sort_by_key, stable_sort_by_key.
//
// As in the reference, sort is implemented as stable_sort on every system
// (thrust/system/detail/generic/sort.inl:57-64).  The device system takes the radix path
// for arithmetic keys with exactly thrust::less or thrust::greater -- the reference's own
// condition for its primitive sort (thrust/system/detail/sequential/sort.inl:139-148,
// thrust/system/cuda/detail/sort.h:1518-1523).  Every other comparator or key type takes
// the stable merge sort, as in the reference (cuda/detail/sort.h:1278-1322).  Its kernels
// are templates on the comparator, so that path exists in translation units compiled
// with hipcc (the comparator must be callable on the device: __host__ __device__); a
// translation unit compiled by a plain host compiler stops there with a message.
#pragma once
#include <algorithm>
#include <cstdint>
#include <cstring>
#include <numeric>
#include <tuple>
#include <vector>

#include <thrust/find.h>
#include <thrust/functional.h>
#include <thrust/iterator/zip_iterator.h>
#include <thrust/tuple.h>
#include <thrust/system/hip/detail/backend.h>
#include <thrust/system/hip/detail/device_input.h>
#include <thrust/iterator/counting_iterator.h>
#include <thrust/iterator/permutation_iterator.h>
#if defined(__HIPCC__)
#include <thrust/system/hip/detail/merge_sort_kernels.h>
#endif

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
namespace detail {
// The reference's host system sorts arithmetic keys under thrust::less / thrust::greater with
// its radix sort (thrust/system/detail/sequential/sort.inl:139-148), i.e. by the keys' radix
// encoding (stable_radix_sort.inl:52-130): floating-point keys are ordered by their bits, -0.0
// before +0.0 and NaNs beyond the infinities of their sign, where operator< would call them
// equivalent or unordered.  rank() is that encoding; for integers it is the key itself.
template <typename K>
inline K rank(K k, std::false_type) { return k; }
inline std::uint32_t rank(float k, std::true_type) {
  std::uint32_t b;
  std::memcpy(&b, &k, sizeof b);
  return b ^ ((b >> 31) ? 0xFFFFFFFFu : 0x80000000u);
}
inline std::uint64_t rank(double k, std::true_type) {
  std::uint64_t b;
  std::memcpy(&b, &k, sizeof b);
  return b ^ ((b >> 63) ? ~std::uint64_t(0) : (std::uint64_t(1) << 63));
}
template <typename K>
struct has_bit_rank : std::integral_constant<bool, std::is_same<K, float>::value || std::is_same<K, double>::value> {};

// CODE: 0 = thrust::less<K>, 1 = thrust::greater<K> on an arithmetic K, < 0 anything else
template <int CODE, typename K, typename Comp>
struct key_order {
  mutable Comp comp;
  bool operator()(const K& a, const K& b) const { return comp(a, b); }
};
template <typename K, typename Comp>
struct key_order<0, K, Comp> {
  mutable Comp comp;
  bool operator()(const K& a, const K& b) const { return rank(a, has_bit_rank<K>()) < rank(b, has_bit_rank<K>()); }
};
template <typename K, typename Comp>
struct key_order<1, K, Comp> {
  mutable Comp comp;
  bool operator()(const K& a, const K& b) const { return rank(b, has_bit_rank<K>()) < rank(a, has_bit_rank<K>()); }
};
template <typename K, typename Comp>
key_order<(!std::is_arithmetic<K>::value ? -1
           : std::is_same<Comp, thrust::less<K> >::value ? 0
           : std::is_same<Comp, thrust::greater<K> >::value ? 1 : -1), K, Comp>
order_of(Comp comp) {
  return {comp};
}
}  // namespace detail

template <typename D, typename It, typename Comp>
void stable_sort(execution_policy<D>&, It first, It last, Comp comp) {
  typedef typename std::remove_const<typename iterator_value<It>::type>::type K;
  std::stable_sort(first, last, detail::order_of<K>(comp));
}
template <typename D, typename KIt, typename VIt, typename Comp>
void stable_sort_by_key(execution_policy<D>&, KIt kf, KIt kl, VIt vf, Comp comp) {
  typedef typename iterator_value<KIt>::type K;
  typedef typename iterator_value<VIt>::type V;
  const std::size_t n = (std::size_t)(kl - kf);
  const auto before = detail::order_of<K>(comp);
  std::vector<std::size_t> order(n);
  std::iota(order.begin(), order.end(), std::size_t(0));
  std::stable_sort(order.begin(), order.end(), [&](std::size_t a, std::size_t b) { return before(kf[a], kf[b]); });
  std::vector<K> k(n);
  std::vector<V> v(n);
  for (std::size_t i = 0; i < n; ++i) { k[i] = kf[order[i]]; v[i] = vf[order[i]]; }
  std::copy(k.begin(), k.end(), kf);
  std::copy(v.begin(), v.end(), vf);
}
}  // namespace cpp

namespace hip {
namespace detail {
// true: arithmetic key ordered by thrust::less / thrust::greater -> radix sort through the C ABI
template <typename K, typename Comp, bool = is_abi_type<K>::value>
struct takes_radix_path : std::integral_constant<bool, (order_code<Comp, K>::value >= 0)> {};
template <typename K, typename Comp>
struct takes_radix_path<K, Comp, false> : std::false_type {};

template <typename T>
struct needs_hipcc : std::false_type {};

// Values travel as opaque items of 1, 2, 4 or 8 bytes: arithmetic types, small structs, and tuples
// of such (a tuple of values is moved bit by bit although its assignment operator is user-written).
template <typename V>
struct is_plain_tuple : std::false_type {};
template <typename... Ts>
struct is_plain_tuple<thrust::tuple<Ts...> >
    : std::integral_constant<bool, std::is_trivially_copyable<std::tuple<Ts...> >::value> {};
template <typename V>
struct is_sort_payload
    : std::integral_constant<bool, (is_abi_item<V>::value || is_plain_tuple<V>::value) &&
                                       (sizeof(V) == 1 || sizeof(V) == 2 || sizeof(V) == 4 || sizeof(V) == 8)> {};
template <typename K, typename V, typename Comp>
struct pairs_take_radix_path
    : std::integral_constant<bool, takes_radix_path<K, Comp>::value && is_sort_payload<V>::value> {};

template <typename K, typename Comp>
void sort_keys(void* stream, temp_source source, K* keys, uint64_t n, Comp, std::true_type) {
  temp_storage temp(stream, source);
  run(temp, 0, "sort failed", [&](void* t, std::size_t* b) {
    return thrust_amd_sort_keys(t, b, keys, n, dtype_of<K>::value, order_code<Comp, K>::value, 0,
                                (int)sizeof(K) * 8, stream);
  });
}
template <typename K, typename V, typename Comp>
void sort_pairs(void* stream, temp_source source, K* keys, V* values, uint64_t n, Comp, std::true_type) {
  temp_storage temp(stream, source);
  run(temp, 0, "sort_by_key failed", [&](void* t, std::size_t* b) {
    return thrust_amd_sort_pairs(t, b, keys, values, n, dtype_of<K>::value, sizeof(V), order_code<Comp, K>::value, 0,
                                 (int)sizeof(K) * 8, stream);
  });
}
#if defined(__HIPCC__)
// The merge sort holds tiles of keys and values in registers and LDS: key and value together
// may take 32 bytes.  Wider elements are sorted through their positions: the merge sort orders
// 32-bit indices by the keys they point at (which stay where they are), and the keys and
// values are gathered into that order afterwards.  The reference's merge sort moves the wide
// elements themselves in every pass (thrust/system/cuda/detail/sort.h:1005-1200).
constexpr std::size_t MERGE_SORT_ITEM_BYTES = 32;
template <typename K, typename Comp>
struct compares_positions {
  const K* keys;
  mutable Comp comp;  // a caller's comparator need not be const-callable
  __host__ __device__ bool operator()(uint32_t a, uint32_t b) const { return comp(keys[a], keys[b]) ? true : false; }
};
template <typename T>
inline void gather_in_place(void* stream, const temp_source& source, T* data, const uint32_t* order, uint64_t n) {
  temp_storage gathered(stream, source);
  gathered.ensure((std::size_t)n * sizeof(T));
  T* out = static_cast<T*>(gathered.ptr());
  materialize(stream, thrust::make_permutation_iterator((const T*)data, order), out, n);
  throw_on_error(thrust_amd_memcpy(data, out, n * sizeof(T), THRUST_AMD_D2D, stream), "sort: copy of the gathered elements");
  synchronize(stream, "sort: synchronize");  // `gathered` returns to the arena when this function ends
}
// positions 0 .. n-1 ordered by keys[position] under comp, stable
template <typename K, typename Comp>
inline void sort_positions(void* stream, const temp_source& source, const K* keys, uint32_t* order, uint64_t n, Comp comp) {
  if (n >= 0xffffffffull) throw thrust::system::system_error((int)hipErrorInvalidValue, "sort of wide elements: positions are 32-bit");
  materialize(stream, thrust::counting_iterator<uint32_t>(0), order, n);
  temp_storage temp(stream, source);
  const compares_positions<K, Comp> by_key = {keys, comp};
  run(temp, 0, "sort (comparison path, wide elements) failed", [&](void* t, std::size_t* b) {
    return thrust::system::hip::merge_sort::sort<uint32_t, unsigned, false>(t, b, order, (unsigned*)nullptr, n, by_key,
                                                                            (hipStream_t)stream);
  });
  synchronize(stream, "sort: synchronize");
}

template <typename K, typename Comp>
void sort_keys_comparing(void* stream, temp_source source, K* keys, uint64_t n, Comp comp, std::true_type /*fits*/) {
  temp_storage temp(stream, source);
  run(temp, 0, "sort (comparison path) failed", [&](void* t, std::size_t* b) {
    return thrust::system::hip::merge_sort::sort<K, unsigned, false>(t, b, keys, (unsigned*)nullptr, n, comp,
                                                                     (hipStream_t)stream);
  });
}
template <typename K, typename Comp>
void sort_keys_comparing(void* stream, temp_source source, K* keys, uint64_t n, Comp comp, std::false_type) {
  temp_storage positions(stream, source);
  positions.ensure((std::size_t)n * sizeof(uint32_t));
  uint32_t* order = static_cast<uint32_t*>(positions.ptr());
  sort_positions(stream, source, (const K*)keys, order, n, comp);
  gather_in_place(stream, source, keys, order, n);
}
template <typename K, typename Comp>
void sort_keys(void* stream, temp_source source, K* keys, uint64_t n, Comp comp, std::false_type) {
  sort_keys_comparing(stream, source, keys, n, comp,
                      std::integral_constant<bool, sizeof(K) <= MERGE_SORT_ITEM_BYTES>());
}

template <typename K, typename V, typename Comp>
void sort_pairs_comparing(void* stream, temp_source source, K* keys, V* values, uint64_t n, Comp comp, std::true_type) {
  temp_storage temp(stream, source);
  run(temp, 0, "sort_by_key (comparison path) failed", [&](void* t, std::size_t* b) {
    return thrust::system::hip::merge_sort::sort<K, V, true>(t, b, keys, values, n, comp, (hipStream_t)stream);
  });
}
template <typename K, typename V, typename Comp>
void sort_pairs_comparing(void* stream, temp_source source, K* keys, V* values, uint64_t n, Comp comp, std::false_type) {
  temp_storage positions(stream, source);
  positions.ensure((std::size_t)n * sizeof(uint32_t));
  uint32_t* order = static_cast<uint32_t*>(positions.ptr());
  sort_positions(stream, source, (const K*)keys, order, n, comp);
  gather_in_place(stream, source, keys, order, n);
  gather_in_place(stream, source, values, order, n);
}
template <typename K, typename V, typename Comp>
void sort_pairs(void* stream, temp_source source, K* keys, V* values, uint64_t n, Comp comp, std::false_type) {
  sort_pairs_comparing(stream, source, keys, values, n, comp,
                       std::integral_constant<bool, sizeof(K) + sizeof(V) <= MERGE_SORT_ITEM_BYTES>());
}
#else
template <typename K, typename Comp>
void sort_keys(void*, temp_source, K*, uint64_t, Comp, std::false_type) {
  static_assert(needs_hipcc<Comp>::value,
                "sort on the device system: comparators other than thrust::less / thrust::greater of an arithmetic "
                "key run as kernels instantiated for the comparator; compile this translation unit with hipcc");
}
template <typename K, typename V, typename Comp>
void sort_pairs(void*, temp_source, K*, V*, uint64_t, Comp, std::false_type) {
  static_assert(needs_hipcc<Comp>::value,
                "sort_by_key on the device system: comparators other than thrust::less / thrust::greater of an "
                "arithmetic key run as kernels instantiated for the comparator; compile this translation unit with hipcc");
}
#endif
}  // namespace detail

namespace detail {
// The array a sort works on.  Device pointers are sorted where they lie; a zip_iterator
// (structure of arrays) is gathered into an array of tuples first and written back through
// the zip afterwards.
template <typename It, bool Fancy = thrust::detail::is_fancy_iterator<It>::value>
class sortable_range {
 public:
  typedef typename iterator_value<It>::type value_type;
  sortable_range(void*, const temp_source&, It first, uint64_t) : ptr_(thrust::detail::raw(first)) {}
  value_type* ptr() const { return ptr_; }
  void write_back() {}

 private:
  value_type* ptr_;
};
template <typename It>
class sortable_range<It, true> {
 public:
  typedef typename iterator_value<It>::type value_type;
  sortable_range(void* stream, const temp_source& source, It first, uint64_t n)
      : holder_(stream, source), stream_(stream), first_(first), n_(n), ptr_(nullptr) {
    static_assert(is_device_output<It>::value,
                  "sort on the device system: a fancy iterator to sort through must be a zip of device iterators");
    holder_.ensure((std::size_t)n * sizeof(value_type));
    ptr_ = static_cast<value_type*>(holder_.ptr());
    materialize(stream, first, ptr_, n);
  }
  value_type* ptr() const { return ptr_; }
  void write_back() { materialize(stream_, (const value_type*)ptr_, first_, n_); }

 private:
  temp_storage holder_;
  void* stream_;
  It first_;
  uint64_t n_;
  value_type* ptr_;
};
}  // namespace detail

template <typename D, typename It, typename Comp>
void stable_sort(execution_policy<D>& exec, It first, It last, Comp comp) {
  typedef typename iterator_value<It>::type K;
  static_assert(detail::is_device_output<It>::value,
                "sort on the device system needs device_ptr / device_vector iterators, raw device pointers or a zip of them");
  void* stream = detail::stream_of(exec);
  const uint64_t n = (uint64_t)(last - first);
  if (n < 2) return;
  detail::sortable_range<It> keys(stream, detail::temp_source_of(exec), first, n);
  detail::sort_keys(stream, detail::temp_source_of(exec), keys.ptr(), n, comp, detail::takes_radix_path<K, Comp>());
  keys.write_back();
  detail::synchronize(stream, "sort: synchronize");
}
template <typename D, typename KIt, typename VIt, typename Comp>
void stable_sort_by_key(execution_policy<D>& exec, KIt kf, KIt kl, VIt vf, Comp comp) {
  typedef typename iterator_value<KIt>::type K;
  static_assert(detail::is_device_output<KIt>::value && detail::is_device_output<VIt>::value,
                "sort_by_key on the device system needs device_ptr / device_vector iterators, raw device pointers or "
                "zips of them");
  void* stream = detail::stream_of(exec);
  const uint64_t n = (uint64_t)(kl - kf);
  if (n < 2) return;
  detail::sortable_range<KIt> keys(stream, detail::temp_source_of(exec), kf, n);
  detail::sortable_range<VIt> values(stream, detail::temp_source_of(exec), vf, n);
  typedef typename iterator_value<VIt>::type V;
  detail::sort_pairs(stream, detail::temp_source_of(exec), keys.ptr(), values.ptr(), n, comp,
                     detail::pairs_take_radix_path<K, V, Comp>());
  keys.write_back();
  values.write_back();
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

// ------------------------------------------------------------------ is_sorted, is_sorted_until
// is_sorted_until: the end of the longest sorted prefix, i.e. the first position whose element is
// before its predecessor, `last` if there is none (thrust/system/detail/generic/sort.inl:155-196: a
// find over the range zipped with itself shifted by one; testing/is_sorted_until.cu, is_sorted.cu).
namespace detail {
template <typename Comp>
struct out_of_order {
  mutable Comp comp;  // a caller's comparison need not be const-callable
  template <typename Tuple>
  __host__ __device__ bool operator()(const Tuple& t) const { return comp(thrust::get<1>(t), thrust::get<0>(t)); }
};
}  // namespace detail

template <typename D, typename It, typename Comp>
It is_sorted_until(const detail::execution_policy_base<D>& exec, It first, It last, Comp comp) {
  const std::ptrdiff_t n = last - first;
  if (n < 2) return last;
  auto pairs = thrust::make_zip_iterator(thrust::make_tuple(first, first + 1));
  const detail::out_of_order<Comp> breaks = {comp};
  return first + ((thrust::find_if(exec, pairs, pairs + (n - 1), breaks) - pairs) + 1);
}
template <typename D, typename It>
It is_sorted_until(const detail::execution_policy_base<D>& exec, It first, It last) {
  typedef typename std::remove_const<typename iterator_value<It>::type>::type V;
  return thrust::is_sorted_until(exec, first, last, thrust::less<V>());
}
template <typename It, typename Comp, typename = typename std::enable_if<!detail::is_execution_policy<It>::value>::type>
It is_sorted_until(It first, It last, Comp comp) {
  return thrust::is_sorted_until(detail::policy_for<It>(), first, last, comp);
}
template <typename It>
It is_sorted_until(It first, It last) {
  return thrust::is_sorted_until(detail::policy_for<It>(), first, last);
}
template <typename D, typename It, typename Comp>
bool is_sorted(const detail::execution_policy_base<D>& exec, It first, It last, Comp comp) {
  return thrust::is_sorted_until(exec, first, last, comp) == last;
}
template <typename D, typename It>
bool is_sorted(const detail::execution_policy_base<D>& exec, It first, It last) {
  return thrust::is_sorted_until(exec, first, last) == last;
}
template <typename It, typename Comp, typename = typename std::enable_if<!detail::is_execution_policy<It>::value>::type>
bool is_sorted(It first, It last, Comp comp) {
  return thrust::is_sorted(detail::policy_for<It>(), first, last, comp);
}
template <typename It>
bool is_sorted(It first, It last) {
  return thrust::is_sorted(detail::policy_for<It>(), first, last);
}

}  // namespace thrust
