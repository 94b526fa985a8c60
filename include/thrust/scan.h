// thrust::inclusive_scan and thrust::exclusive_scan.
//
// Accumulator types follow the reference (thrust/system/detail/sequential/scan.h:48-115,
// P0571): inclusive scans accumulate in the input's value type, exclusive scans in the
// type of init; exclusive_scan(first,last,result) uses init = value_type(0); the default
// operator is plus (thrust/system/detail/generic/scan.inl:39-81).  In-place is allowed.
//
// thrust::inclusive_scan_by_key and thrust::exclusive_scan_by_key scan every run of
// consecutive equal keys on its own (thrust/system/detail/generic/scan_by_key.inl:62-238):
// default key predicate equal_to, default operator plus, default init value_type{}; the
// exclusive form yields init at the first element of every run.
#pragma once
#include <thrust/functional.h>
#include <thrust/system/hip/detail/backend.h>
#include <thrust/system/hip/detail/device_input.h>
#include <thrust/system/hip/detail/staged_output.h>
#if defined(__HIPCC__)
#include <thrust/system/hip/detail/generic_kernels.h>
#include <thrust/system/hip/detail/generic_select.h>
#include <thrust/system/hip/detail/scan_kernels.h>
#endif

namespace thrust {

template <typename D, typename In, typename Out>
Out inclusive_scan(const detail::execution_policy_base<D>& exec, In first, In last, Out result);
template <typename D, typename In, typename Out, typename Op>
Out inclusive_scan(const detail::execution_policy_base<D>& exec, In first, In last, Out result, Op op);
template <typename D, typename In, typename Out>
Out exclusive_scan(const detail::execution_policy_base<D>& exec, In first, In last, Out result);
template <typename D, typename In, typename Out, typename T>
Out exclusive_scan(const detail::execution_policy_base<D>& exec, In first, In last, Out result, T init);
template <typename D, typename In, typename Out, typename T, typename Op>
Out exclusive_scan(const detail::execution_policy_base<D>& exec, In first, In last, Out result, T init, Op op);

template <typename D, typename KIt, typename VIt, typename Out>
Out inclusive_scan_by_key(const detail::execution_policy_base<D>& exec, KIt kf, KIt kl, VIt vf, Out result);
template <typename D, typename KIt, typename VIt, typename Out, typename Pred>
Out inclusive_scan_by_key(const detail::execution_policy_base<D>& exec, KIt kf, KIt kl, VIt vf, Out result, Pred pred);
template <typename D, typename KIt, typename VIt, typename Out, typename Pred, typename Op>
Out inclusive_scan_by_key(const detail::execution_policy_base<D>& exec, KIt kf, KIt kl, VIt vf, Out result, Pred pred,
                          Op op);
template <typename D, typename KIt, typename VIt, typename Out>
Out exclusive_scan_by_key(const detail::execution_policy_base<D>& exec, KIt kf, KIt kl, VIt vf, Out result);
template <typename D, typename KIt, typename VIt, typename Out, typename T>
Out exclusive_scan_by_key(const detail::execution_policy_base<D>& exec, KIt kf, KIt kl, VIt vf, Out result, T init);
template <typename D, typename KIt, typename VIt, typename Out, typename T, typename Pred>
Out exclusive_scan_by_key(const detail::execution_policy_base<D>& exec, KIt kf, KIt kl, VIt vf, Out result, T init,
                          Pred pred);
template <typename D, typename KIt, typename VIt, typename Out, typename T, typename Pred, typename Op>
Out exclusive_scan_by_key(const detail::execution_policy_base<D>& exec, KIt kf, KIt kl, VIt vf, Out result, T init,
                          Pred pred, Op op);

namespace system {
namespace detail {
namespace generic {
template <typename D, typename KIt, typename VIt, typename Out>
Out inclusive_scan_by_key(thrust::execution_policy<D>& exec, KIt kf, KIt kl, VIt vf, Out result) {
  return thrust::inclusive_scan_by_key(exec, kf, kl, vf, result, thrust::equal_to<>());
}
template <typename D, typename KIt, typename VIt, typename Out, typename Pred>
Out inclusive_scan_by_key(thrust::execution_policy<D>& exec, KIt kf, KIt kl, VIt vf, Out result, Pred pred) {
  return thrust::inclusive_scan_by_key(exec, kf, kl, vf, result, pred, thrust::plus<>());
}
template <typename D, typename KIt, typename VIt, typename Out>
Out exclusive_scan_by_key(thrust::execution_policy<D>& exec, KIt kf, KIt kl, VIt vf, Out result) {
  typedef typename iterator_value<VIt>::type T;
  return thrust::exclusive_scan_by_key(exec, kf, kl, vf, result, T());
}
template <typename D, typename KIt, typename VIt, typename Out, typename T>
Out exclusive_scan_by_key(thrust::execution_policy<D>& exec, KIt kf, KIt kl, VIt vf, Out result, T init) {
  return thrust::exclusive_scan_by_key(exec, kf, kl, vf, result, init, thrust::equal_to<>());
}
template <typename D, typename KIt, typename VIt, typename Out, typename T, typename Pred>
Out exclusive_scan_by_key(thrust::execution_policy<D>& exec, KIt kf, KIt kl, VIt vf, Out result, T init, Pred pred) {
  return thrust::exclusive_scan_by_key(exec, kf, kl, vf, result, init, pred, thrust::plus<>());
}
template <typename D, typename In, typename Out>
Out inclusive_scan(thrust::execution_policy<D>& exec, In first, In last, Out result) {
  return thrust::inclusive_scan(exec, first, last, result, thrust::plus<>());
}
template <typename D, typename In, typename Out>
Out exclusive_scan(thrust::execution_policy<D>& exec, In first, In last, Out result) {
  typedef typename iterator_value<In>::type T;
  return thrust::exclusive_scan(exec, first, last, result, T(0));
}
template <typename D, typename In, typename Out, typename T>
Out exclusive_scan(thrust::execution_policy<D>& exec, In first, In last, Out result, T init) {
  return thrust::exclusive_scan(exec, first, last, result, init, thrust::plus<>());
}
}  // namespace generic
}  // namespace detail

namespace cpp {
template <typename D, typename In, typename Out, typename Op>
Out inclusive_scan(execution_policy<D>&, In first, In last, Out result, Op op) {
  typedef typename iterator_value<In>::type T;
  if (first != last) {
    T sum = *first;
    *result = sum;
    for (++first, ++result; first != last; ++first, ++result) *result = sum = op(sum, *first);
  }
  return result;
}
template <typename D, typename In, typename Out, typename T, typename Op>
Out exclusive_scan(execution_policy<D>&, In first, In last, Out result, T init, Op op) {
  if (first != last) {
    T tmp = *first;
    T sum = init;
    *result = sum;
    sum = op(sum, tmp);
    for (++first, ++result; first != last; ++first, ++result) {
      tmp = *first;
      *result = sum;
      sum = op(sum, tmp);
    }
  }
  return result;
}
// Sequential segmented scans (thrust/system/detail/sequential/scan_by_key.h:38-145).
template <typename D, typename KIt, typename VIt, typename Out, typename Pred, typename Op>
Out inclusive_scan_by_key(execution_policy<D>&, KIt kf, KIt kl, VIt vf, Out result, Pred pred, Op op) {
  typedef typename iterator_value<KIt>::type K;
  typedef typename iterator_value<VIt>::type V;
  if (kf != kl) {
    K prev_key = *kf;
    V prev_value = *vf;
    *result = prev_value;
    for (++kf, ++vf, ++result; kf != kl; ++kf, ++vf, ++result) {
      const K key = *kf;
      if (pred(prev_key, key)) *result = prev_value = op(prev_value, *vf);
      else *result = prev_value = *vf;
      prev_key = key;
    }
  }
  return result;
}
template <typename D, typename KIt, typename VIt, typename Out, typename T, typename Pred, typename Op>
Out exclusive_scan_by_key(execution_policy<D>&, KIt kf, KIt kl, VIt vf, Out result, T init, Pred pred, Op op) {
  typedef typename iterator_value<KIt>::type K;
  if (kf != kl) {
    K temp_key = *kf;
    T temp_value = *vf;
    T next = init;
    *result = next;
    next = op(next, temp_value);
    for (++kf, ++vf, ++result; kf != kl; ++kf, ++vf, ++result) {
      const K key = *kf;
      temp_value = *vf;  // read before the write: in place is allowed
      if (!pred(temp_key, key)) next = init;
      *result = next;
      next = op(next, temp_value);
      temp_key = key;
    }
  }
  return result;
}
}  // namespace cpp

namespace hip {
// The accumulator's type is the input's element type for inclusive_scan and the type of init
// for exclusive_scan; input and output may hold other arithmetic types, converted on the way
// in and out as the reference does (testing/scan.cu:236-295).
namespace detail {
template <typename D, typename In, typename Out, typename Op>
Out inclusive_scan(execution_policy<D>& exec, In first, In last, Out result, Op, std::true_type) {
  typedef typename std::remove_const<typename iterator_value<In>::type>::type V;
  typedef typename iterator_value<Out>::type U;
  void* stream = stream_of(exec);
  const uint64_t n = (uint64_t)(last - first);
  if (n == 0) return result;
  device_input<In> source(stream, temp_source_of(exec), first, n);
  temp_storage staged(stream, temp_source_of(exec));
  V* computed = output_as<V>(static_cast<U*>(thrust::detail::raw(result)), n, staged);
  temp_storage temp(stream, temp_source_of(exec));
  run(temp, 0, "inclusive_scan failed", [&](void* t, std::size_t* b) {
    return thrust_amd_inclusive_scan(t, b, source.ptr(), computed, n, dtype_of<V>::value,
                                     binop_code<Op, V>::value, stream);
  });
  finish_output(computed, static_cast<U*>(thrust::detail::raw(result)), n, stream);
  synchronize(stream, "inclusive_scan: synchronize");
  return result + n;
}

template <typename D, typename In, typename Out, typename T, typename Op>
Out exclusive_scan(execution_policy<D>& exec, In first, In last, Out result, T init, Op, std::true_type) {
  typedef typename iterator_value<Out>::type U;
  void* stream = stream_of(exec);
  const uint64_t n = (uint64_t)(last - first);
  if (n == 0) return result;
  device_input<In> source(stream, temp_source_of(exec), first, n);
  temp_storage converted(stream, temp_source_of(exec));
  const T* in = input_as<T>(source.ptr(), n, stream, converted);
  temp_storage staged(stream, temp_source_of(exec));
  T* computed = output_as<T>(static_cast<U*>(thrust::detail::raw(result)), n, staged);
  temp_storage temp(stream, temp_source_of(exec));
  run(temp, 0, "exclusive_scan failed", [&](void* t, std::size_t* b) {
    return thrust_amd_exclusive_scan(t, b, in, computed, n, dtype_of<T>::value,
                                     binop_code<Op, T>::value, &init, stream);
  });
  finish_output(computed, static_cast<U*>(thrust::detail::raw(result)), n, stream);
  synchronize(stream, "exclusive_scan: synchronize");
  return result + n;
}

// A user's operator or element type: three kernels instantiated for them (hipcc translation
// units).  A is the accumulator's type, as in the library path.
template <bool EXCLUSIVE, typename A, typename D, typename In, typename Out, typename Op>
Out scan_generic(execution_policy<D>& exec, In first, In last, Out result, A init, Op op) {
  static_assert(is_device_input<In>::value && is_device_output<Out>::value,
                "scan on the device system needs device_ptr / device_vector iterators, raw device pointers, fancy "
                "iterators, or for the output an iterator type that kernels can take by value");
#if defined(__HIPCC__)
  namespace gk = thrust::system::hip::generic;
  typedef typename thrust::detail::device_view_of<In>::type View;
  typedef typename thrust::detail::device_view_of<Out>::type OutView;
  typedef typename thrust::detail::output_value<Out, A>::type U;
  void* stream = stream_of(exec);
  const uint64_t n = (uint64_t)(last - first);
  if (n == 0) return result;
  constexpr uint64_t TILE = gk::scan_shape<A>::TILE;
  const uint64_t tiles = (n + TILE - 1) / TILE;
  if (tiles > 0xffffffffull) throw_on_error(1, "scan: range too long");
  // The tile totals are scanned in place: by one workgroup when there are few, otherwise by the
  // same three steps one level up (their tile totals, scanned, then every tile of totals on top
  // of what precedes it).  level[k] holds the totals of level k - 1's tiles; level[0] those of the input.
  constexpr uint64_t ONE_WORKGROUP = 4 * gk::BLOCK;
  constexpr int MAX_LEVELS = 8;
  uint64_t count[MAX_LEVELS];
  std::size_t offset[MAX_LEVELS];
  int levels = 0;
  std::size_t bytes = 0;
  for (uint64_t c = tiles;; c = (c + TILE - 1) / TILE) {
    count[levels] = c;
    offset[levels] = bytes;
    bytes += ((std::size_t)c * sizeof(A) + 255) / 256 * 256;
    ++levels;
    if (c <= ONE_WORKGROUP || levels == MAX_LEVELS) break;
  }
  temp_storage temp(stream, temp_source_of(exec));
  temp.ensure(bytes);
  A* level[MAX_LEVELS];
  for (int k = 0; k < levels; ++k) level[k] = reinterpret_cast<A*>(static_cast<char*>(temp.ptr()) + offset[k]);
  A* tile_total = level[0];
  hipLaunchKernelGGL((gk::scan_tile_totals_kernel<View, A, Op>), dim3((unsigned)tiles), dim3(gk::BLOCK), 0,
                     (hipStream_t)stream, thrust::detail::device_view(first), n, op, tile_total);
  throw_on_error(launch_status(), "scan: kernel launch");
  for (int k = 1; k < levels; ++k) {
    hipLaunchKernelGGL((gk::scan_tile_totals_kernel<const A*, A, Op>), dim3((unsigned)count[k]), dim3(gk::BLOCK), 0,
                       (hipStream_t)stream, (const A*)level[k - 1], count[k - 1], op, level[k]);
    throw_on_error(launch_status(), "scan: kernel launch");
  }
  hipLaunchKernelGGL((gk::scan_tile_prefix_kernel<A, Op>), dim3(1), dim3(gk::BLOCK), 0, (hipStream_t)stream,
                     level[levels - 1], (uint32_t)count[levels - 1], op);
  throw_on_error(launch_status(), "scan: kernel launch");
  for (int k = levels - 1; k >= 1; --k) {
    // in place: a workgroup reads its tile into registers before it writes
    hipLaunchKernelGGL((gk::scan_tiles_kernel<false, const A*, A, A, A*, Op>), dim3((unsigned)count[k]), dim3(gk::BLOCK), 0,
                       (hipStream_t)stream, (const A*)level[k - 1], level[k - 1], count[k - 1], op, init,
                       (const A*)level[k]);
    throw_on_error(launch_status(), "scan: kernel launch");
  }
  hipLaunchKernelGGL((gk::scan_tiles_kernel<EXCLUSIVE, View, A, U, OutView, Op>), dim3((unsigned)tiles), dim3(gk::BLOCK), 0,
                     (hipStream_t)stream, thrust::detail::device_view(first), thrust::detail::device_view(result), n, op, init,
                     (const A*)tile_total);
  throw_on_error(launch_status(), "scan: kernel launch");
  synchronize(stream, "scan: synchronize");
  return result + n;
#else
  static_assert(fancy_needs_hipcc<Op>::value,
                "scan on the device system: operators other than thrust::plus / minimum / maximum of an arithmetic "
                "type run in kernels instantiated for the operator; compile this translation unit with hipcc");
  return result;
#endif
}
#if defined(__HIPCC__)
// Elements of 4 or 8 bytes, the same type in, out and in the accumulator, written to device
// memory: the single-pass scan (scan_kernels.h), instantiated for the operator.  Everything
// else (wider structs, converting scans, outputs that are not memory) takes scan_generic.
template <typename A, typename In, typename Out>
struct scans_in_one_pass
    : std::integral_constant<bool, is_kernel_item<A>::value && (sizeof(A) == 4 || sizeof(A) == 8) &&
                                       std::is_same<typename std::remove_const<typename iterator_value<In>::type>::type, A>::value &&
                                       std::is_same<typename iterator_value<Out>::type, A>::value &&
                                       (std::is_pointer<Out>::value || thrust::detail::is_device_iterator<Out>::value)> {};
template <bool EXCLUSIVE, typename A, typename D, typename In, typename Out, typename Op>
Out scan_one_pass(execution_policy<D>& exec, In first, In last, Out result, A init, Op op) {
  namespace sc = thrust::system::hip::scanning;
  void* stream = stream_of(exec);
  const uint64_t n = (uint64_t)(last - first);
  if (n == 0) return result;
  device_input<In> source(stream, temp_source_of(exec), first, n);
  temp_storage temp(stream, temp_source_of(exec));
  temp.ensure(sc::scan_temp_bytes<A>(n));
  throw_on_error(sc::ordered_scan_launch<EXCLUSIVE>(static_cast<char*>(temp.ptr()), (const A*)source.ptr(),
                                                    (A*)thrust::detail::raw(result), n, init, op, (hipStream_t)stream),
                 "scan failed");
  synchronize(stream, "scan: synchronize");
  return result + n;
}
template <bool EXCLUSIVE, typename A, typename D, typename In, typename Out, typename Op>
Out scan_user(execution_policy<D>& exec, In first, In last, Out result, A init, Op op, std::true_type) {
  return scan_one_pass<EXCLUSIVE, A>(exec, first, last, result, init, op);
}
#endif
template <bool EXCLUSIVE, typename A, typename D, typename In, typename Out, typename Op>
Out scan_user(execution_policy<D>& exec, In first, In last, Out result, A init, Op op, std::false_type) {
  return scan_generic<EXCLUSIVE, A>(exec, first, last, result, init, op);
}
template <typename A, typename In, typename Out>
struct scan_user_route
#if defined(__HIPCC__)
    : scans_in_one_pass<A, In, Out> {
};
#else
    : std::false_type {
};
#endif
template <typename D, typename In, typename Out, typename Op>
Out inclusive_scan(execution_policy<D>& exec, In first, In last, Out result, Op op, std::false_type) {
  typedef typename std::remove_const<typename iterator_value<In>::type>::type V;
  return scan_user<false, V>(exec, first, last, result, V(), op, scan_user_route<V, In, Out>());
}
template <typename D, typename In, typename Out, typename T, typename Op>
Out exclusive_scan(execution_policy<D>& exec, In first, In last, Out result, T init, Op op, std::false_type) {
  return scan_user<true, T>(exec, first, last, result, init, op, scan_user_route<T, In, Out>());
}

// library path: arithmetic input, output and accumulator with plus / minimum / maximum of the accumulator's type
template <typename V, typename U, typename A, typename Op,
          bool = is_abi_type<V>::value && is_abi_type<U>::value && is_abi_type<A>::value>
struct scans_in_library : std::integral_constant<bool, (binop_code<Op, A>::value >= 0)> {};
template <typename V, typename U, typename A, typename Op>
struct scans_in_library<V, U, A, Op, false> : std::false_type {};
}  // namespace detail

template <typename D, typename In, typename Out, typename Op>
Out inclusive_scan(execution_policy<D>& exec, In first, In last, Out result, Op op) {
  typedef typename std::remove_const<typename iterator_value<In>::type>::type V;
  typedef typename iterator_value<Out>::type U;
  // the library's kernels write arrays; any other output (an iterator type of the caller's own,
  // discard_iterator) is written by the generic kernels, which take it by value
  typedef std::integral_constant<bool, detail::scans_in_library<V, U, V, Op>::value &&
                                           (std::is_pointer<Out>::value || thrust::detail::is_device_iterator<Out>::value)> in_library;
  return detail::inclusive_scan(exec, first, last, result, op, in_library());
}
template <typename D, typename In, typename Out, typename T, typename Op>
Out exclusive_scan(execution_policy<D>& exec, In first, In last, Out result, T init, Op op) {
  typedef typename std::remove_const<typename iterator_value<In>::type>::type V;
  typedef typename iterator_value<Out>::type U;
  typedef std::integral_constant<bool, detail::scans_in_library<V, U, T, Op>::value &&
                                           (std::is_pointer<Out>::value || thrust::detail::is_device_iterator<Out>::value)> in_library;
  return detail::exclusive_scan(exec, first, last, result, init, op, in_library());
}

namespace detail {
template <typename KIt, typename VIt, typename Out, typename T, typename Pred, typename Op>
struct scan_by_key_checks {
  typedef typename std::remove_const<typename iterator_value<KIt>::type>::type K;
  typedef typename std::remove_const<typename iterator_value<VIt>::type>::type V;
  static_assert((std::is_pointer<KIt>::value || thrust::detail::is_device_iterator<KIt>::value) &&
                    (std::is_pointer<VIt>::value || thrust::detail::is_device_iterator<VIt>::value) &&
                    (std::is_pointer<Out>::value || thrust::detail::is_device_iterator<Out>::value),
                "scan_by_key on the device system needs device_ptr / device_vector iterators or raw device pointers");
  static_assert(is_abi_type<K>::value && is_abi_type<V>::value && std::is_same<V, T>::value &&
                    std::is_same<typename iterator_value<Out>::type, V>::value,
                "scan_by_key on the device system: arithmetic keys; values, output and init share one arithmetic type");
  static_assert(is_equal_to<Pred, K>::value,
                "scan_by_key on the device system supports thrust::equal_to as key predicate");
  static_assert(binop_code<Op, V>::value >= 0,
                "scan_by_key on the device system supports thrust::plus, thrust::minimum and thrust::maximum");
};
}  // namespace detail

namespace detail {
// library path: arithmetic keys and values of one type, equal_to, plus / minimum / maximum
template <typename K, typename V, typename U, typename T, typename Pred, typename Op,
          bool = is_abi_type<K>::value && is_abi_type<V>::value && std::is_same<V, T>::value && std::is_same<U, V>::value>
struct scans_by_key_in_library
    : std::integral_constant<bool, is_equal_to<Pred, K>::value && (binop_code<Op, V>::value >= 0)> {};
template <typename K, typename V, typename U, typename T, typename Pred, typename Op>
struct scans_by_key_in_library<K, V, U, T, Pred, Op, false> : std::false_type {};

// a user's key predicate, operator or element types (defined with the other by-key pieces,
// in translation units compiled with hipcc)
template <bool EXCLUSIVE, typename D, typename KIt, typename VIt, typename Out, typename A, typename Pred, typename Op>
Out scan_by_key_generic(execution_policy<D>& exec, KIt kf, KIt kl, VIt vf, Out result, A init, Pred pred, Op op);
}  // namespace detail

template <typename D, typename KIt, typename VIt, typename Out, typename Pred, typename Op>
Out inclusive_scan_by_key_library(execution_policy<D>& exec, KIt kf, KIt kl, VIt vf, Out result, Pred, Op) {
  typedef detail::scan_by_key_checks<KIt, VIt, Out, typename std::remove_const<typename iterator_value<VIt>::type>::type, Pred, Op> C;
  typedef typename C::K K;
  typedef typename C::V V;
  void* stream = detail::stream_of(exec);
  const uint64_t n = (uint64_t)(kl - kf);
  if (n == 0) return result;
  detail::temp_storage temp(stream, detail::temp_source_of(exec));
  detail::run(temp, 0, "inclusive_scan_by_key failed", [&](void* t, std::size_t* b) {
    return thrust_amd_inclusive_scan_by_key(t, b, thrust::detail::raw(kf), thrust::detail::raw(vf),
                                            thrust::detail::raw(result), n, detail::dtype_of<K>::value,
                                            detail::dtype_of<V>::value, detail::binop_code<Op, V>::value, stream);
  });
  detail::synchronize(stream, "inclusive_scan_by_key: synchronize");
  return result + n;
}

template <typename D, typename KIt, typename VIt, typename Out, typename T, typename Pred, typename Op>
Out exclusive_scan_by_key_library(execution_policy<D>& exec, KIt kf, KIt kl, VIt vf, Out result, T init, Pred, Op) {
  typedef detail::scan_by_key_checks<KIt, VIt, Out, T, Pred, Op> C;
  typedef typename C::K K;
  typedef typename C::V V;
  void* stream = detail::stream_of(exec);
  const uint64_t n = (uint64_t)(kl - kf);
  if (n == 0) return result;
  const void* values = thrust::detail::raw(vf);
  void* out = thrust::detail::raw(result);  // may be the values themselves
  detail::temp_storage temp(stream, detail::temp_source_of(exec));
  detail::run(temp, 0, "exclusive_scan_by_key failed", [&](void* t, std::size_t* b) {
    return thrust_amd_exclusive_scan_by_key(t, b, thrust::detail::raw(kf), values, out, n,
                                            detail::dtype_of<K>::value, detail::dtype_of<V>::value,
                                            detail::binop_code<Op, V>::value, &init, stream);
  });
  detail::synchronize(stream, "exclusive_scan_by_key: synchronize");
  return result + n;
}

namespace detail {
template <typename D, typename KIt, typename VIt, typename Out, typename Pred, typename Op>
Out inclusive_scan_by_key(execution_policy<D>& exec, KIt kf, KIt kl, VIt vf, Out result, Pred pred, Op op, std::true_type) {
  return inclusive_scan_by_key_library(exec, kf, kl, vf, result, pred, op);
}
template <typename D, typename KIt, typename VIt, typename Out, typename T, typename Pred, typename Op>
Out exclusive_scan_by_key(execution_policy<D>& exec, KIt kf, KIt kl, VIt vf, Out result, T init, Pred pred, Op op,
                          std::true_type) {
  return exclusive_scan_by_key_library(exec, kf, kl, vf, result, init, pred, op);
}
#if defined(__HIPCC__)
template <typename D, typename KIt, typename VIt, typename Out, typename Pred, typename Op>
Out inclusive_scan_by_key(execution_policy<D>& exec, KIt kf, KIt kl, VIt vf, Out result, Pred pred, Op op, std::false_type) {
  typedef typename std::remove_const<typename iterator_value<VIt>::type>::type V;
  return scan_by_key_generic<false>(exec, kf, kl, vf, result, V(), pred, op);
}
template <typename D, typename KIt, typename VIt, typename Out, typename T, typename Pred, typename Op>
Out exclusive_scan_by_key(execution_policy<D>& exec, KIt kf, KIt kl, VIt vf, Out result, T init, Pred pred, Op op,
                          std::false_type) {
  return scan_by_key_generic<true>(exec, kf, kl, vf, result, init, pred, op);
}
#else
template <typename D, typename KIt, typename VIt, typename Out, typename Pred, typename Op>
Out inclusive_scan_by_key(execution_policy<D>&, KIt, KIt, VIt, Out result, Pred, Op, std::false_type) {
  static_assert(fancy_needs_hipcc<Op>::value,
                "scan_by_key on the device system: key predicates other than thrust::equal_to, operators other than "
                "thrust::plus / minimum / maximum and non-arithmetic elements run in kernels instantiated for them; "
                "compile this translation unit with hipcc");
  return result;
}
template <typename D, typename KIt, typename VIt, typename Out, typename T, typename Pred, typename Op>
Out exclusive_scan_by_key(execution_policy<D>&, KIt, KIt, VIt, Out result, T, Pred, Op, std::false_type) {
  static_assert(fancy_needs_hipcc<Op>::value,
                "scan_by_key on the device system: key predicates other than thrust::equal_to, operators other than "
                "thrust::plus / minimum / maximum and non-arithmetic elements run in kernels instantiated for them; "
                "compile this translation unit with hipcc");
  return result;
}
#endif
}  // namespace detail

template <typename D, typename KIt, typename VIt, typename Out, typename Pred, typename Op>
Out inclusive_scan_by_key(execution_policy<D>& exec, KIt kf, KIt kl, VIt vf, Out result, Pred pred, Op op) {
  typedef typename std::remove_const<typename iterator_value<KIt>::type>::type K;
  typedef typename std::remove_const<typename iterator_value<VIt>::type>::type V;
  // the library's kernels read and write arrays; fancy inputs and outputs that are not memory
  // (discard_iterator, a zip) go through the kernels instantiated for the iterators
  typedef std::integral_constant<bool, detail::scans_by_key_in_library<K, V, typename iterator_value<Out>::type, V, Pred, Op>::value &&
                                           detail::is_memory_iterator<KIt>::value && detail::is_memory_iterator<VIt>::value &&
                                           detail::is_memory_iterator<Out>::value> in_library;
  return detail::inclusive_scan_by_key(exec, kf, kl, vf, result, pred, op, in_library());
}
template <typename D, typename KIt, typename VIt, typename Out, typename T, typename Pred, typename Op>
Out exclusive_scan_by_key(execution_policy<D>& exec, KIt kf, KIt kl, VIt vf, Out result, T init, Pred pred, Op op) {
  typedef typename std::remove_const<typename iterator_value<KIt>::type>::type K;
  typedef typename std::remove_const<typename iterator_value<VIt>::type>::type V;
  typedef std::integral_constant<bool, detail::scans_by_key_in_library<K, V, typename iterator_value<Out>::type, T, Pred, Op>::value &&
                                           detail::is_memory_iterator<KIt>::value && detail::is_memory_iterator<VIt>::value &&
                                           detail::is_memory_iterator<Out>::value> in_library;
  return detail::exclusive_scan_by_key(exec, kf, kl, vf, result, init, pred, op, in_library());
}
}  // namespace hip
}  // namespace system

template <typename D, typename In, typename Out>
Out inclusive_scan(const detail::execution_policy_base<D>& exec, In first, In last, Out result) {
  using thrust::system::detail::generic::inclusive_scan;
  return inclusive_scan(detail::derived_cast(detail::strip_const(exec)), first, last, result);
}
template <typename D, typename In, typename Out, typename Op>
Out inclusive_scan(const detail::execution_policy_base<D>& exec, In first, In last, Out result, Op op) {
  using thrust::system::detail::generic::inclusive_scan;
  return inclusive_scan(detail::derived_cast(detail::strip_const(exec)), first, last, result, op);
}
template <typename D, typename In, typename Out>
Out exclusive_scan(const detail::execution_policy_base<D>& exec, In first, In last, Out result) {
  using thrust::system::detail::generic::exclusive_scan;
  return exclusive_scan(detail::derived_cast(detail::strip_const(exec)), first, last, result);
}
template <typename D, typename In, typename Out, typename T>
Out exclusive_scan(const detail::execution_policy_base<D>& exec, In first, In last, Out result, T init) {
  using thrust::system::detail::generic::exclusive_scan;
  return exclusive_scan(detail::derived_cast(detail::strip_const(exec)), first, last, result, init);
}
template <typename D, typename In, typename Out, typename T, typename Op>
Out exclusive_scan(const detail::execution_policy_base<D>& exec, In first, In last, Out result, T init, Op op) {
  using thrust::system::detail::generic::exclusive_scan;
  return exclusive_scan(detail::derived_cast(detail::strip_const(exec)), first, last, result, init, op);
}

template <typename In, typename Out>
Out inclusive_scan(In first, In last, Out result) {
  return thrust::inclusive_scan(detail::policy_for<In>(), first, last, result);
}
template <typename In, typename Out, typename Op,
          typename = typename std::enable_if<!detail::is_execution_policy<In>::value>::type>
Out inclusive_scan(In first, In last, Out result, Op op) {
  return thrust::inclusive_scan(detail::policy_for<In>(), first, last, result, op);
}
template <typename In, typename Out>
Out exclusive_scan(In first, In last, Out result) {
  return thrust::exclusive_scan(detail::policy_for<In>(), first, last, result);
}
template <typename In, typename Out, typename T,
          typename = typename std::enable_if<!detail::is_execution_policy<In>::value>::type>
Out exclusive_scan(In first, In last, Out result, T init) {
  return thrust::exclusive_scan(detail::policy_for<In>(), first, last, result, init);
}
template <typename In, typename Out, typename T, typename Op,
          typename = typename std::enable_if<!detail::is_execution_policy<In>::value>::type>
Out exclusive_scan(In first, In last, Out result, T init, Op op) {
  return thrust::exclusive_scan(detail::policy_for<In>(), first, last, result, init, op);
}


#define THRUST_AMD_SCAN_BY_KEY_ENTRY(NAME, TPARAMS, PARAMS, ARGS)                                                  \
  template <typename D, typename KIt, typename VIt, typename Out TPARAMS>                                          \
  Out NAME(const detail::execution_policy_base<D>& exec, KIt kf, KIt kl, VIt vf, Out result PARAMS) {              \
    using thrust::system::detail::generic::NAME;                                                                   \
    return NAME(detail::derived_cast(detail::strip_const(exec)), kf, kl, vf, result ARGS);                         \
  }
#define THRUST_AMD_COMMA ,
THRUST_AMD_SCAN_BY_KEY_ENTRY(inclusive_scan_by_key, , , )
THRUST_AMD_SCAN_BY_KEY_ENTRY(inclusive_scan_by_key, THRUST_AMD_COMMA typename Pred, THRUST_AMD_COMMA Pred pred,
                             THRUST_AMD_COMMA pred)
THRUST_AMD_SCAN_BY_KEY_ENTRY(inclusive_scan_by_key, THRUST_AMD_COMMA typename Pred THRUST_AMD_COMMA typename Op,
                             THRUST_AMD_COMMA Pred pred THRUST_AMD_COMMA Op op,
                             THRUST_AMD_COMMA pred THRUST_AMD_COMMA op)
THRUST_AMD_SCAN_BY_KEY_ENTRY(exclusive_scan_by_key, , , )
THRUST_AMD_SCAN_BY_KEY_ENTRY(exclusive_scan_by_key, THRUST_AMD_COMMA typename T, THRUST_AMD_COMMA T init,
                             THRUST_AMD_COMMA init)
THRUST_AMD_SCAN_BY_KEY_ENTRY(exclusive_scan_by_key, THRUST_AMD_COMMA typename T THRUST_AMD_COMMA typename Pred,
                             THRUST_AMD_COMMA T init THRUST_AMD_COMMA Pred pred,
                             THRUST_AMD_COMMA init THRUST_AMD_COMMA pred)
THRUST_AMD_SCAN_BY_KEY_ENTRY(exclusive_scan_by_key,
                             THRUST_AMD_COMMA typename T THRUST_AMD_COMMA typename Pred THRUST_AMD_COMMA typename Op,
                             THRUST_AMD_COMMA T init THRUST_AMD_COMMA Pred pred THRUST_AMD_COMMA Op op,
                             THRUST_AMD_COMMA init THRUST_AMD_COMMA pred THRUST_AMD_COMMA op)
#undef THRUST_AMD_SCAN_BY_KEY_ENTRY

// without a policy: the system of the key iterator
template <typename KIt, typename VIt, typename Out,
          typename = typename std::enable_if<!detail::is_execution_policy<KIt>::value>::type>
Out inclusive_scan_by_key(KIt kf, KIt kl, VIt vf, Out result) {
  return thrust::inclusive_scan_by_key(detail::policy_for<KIt>(), kf, kl, vf, result);
}
template <typename KIt, typename VIt, typename Out, typename Pred,
          typename = typename std::enable_if<!detail::is_execution_policy<KIt>::value>::type>
Out inclusive_scan_by_key(KIt kf, KIt kl, VIt vf, Out result, Pred pred) {
  return thrust::inclusive_scan_by_key(detail::policy_for<KIt>(), kf, kl, vf, result, pred);
}
template <typename KIt, typename VIt, typename Out, typename Pred, typename Op,
          typename = typename std::enable_if<!detail::is_execution_policy<KIt>::value>::type>
Out inclusive_scan_by_key(KIt kf, KIt kl, VIt vf, Out result, Pred pred, Op op) {
  return thrust::inclusive_scan_by_key(detail::policy_for<KIt>(), kf, kl, vf, result, pred, op);
}
template <typename KIt, typename VIt, typename Out,
          typename = typename std::enable_if<!detail::is_execution_policy<KIt>::value>::type>
Out exclusive_scan_by_key(KIt kf, KIt kl, VIt vf, Out result) {
  return thrust::exclusive_scan_by_key(detail::policy_for<KIt>(), kf, kl, vf, result);
}
template <typename KIt, typename VIt, typename Out, typename T,
          typename = typename std::enable_if<!detail::is_execution_policy<KIt>::value>::type>
Out exclusive_scan_by_key(KIt kf, KIt kl, VIt vf, Out result, T init) {
  return thrust::exclusive_scan_by_key(detail::policy_for<KIt>(), kf, kl, vf, result, init);
}
template <typename KIt, typename VIt, typename Out, typename T, typename Pred,
          typename = typename std::enable_if<!detail::is_execution_policy<KIt>::value>::type>
Out exclusive_scan_by_key(KIt kf, KIt kl, VIt vf, Out result, T init, Pred pred) {
  return thrust::exclusive_scan_by_key(detail::policy_for<KIt>(), kf, kl, vf, result, init, pred);
}
template <typename KIt, typename VIt, typename Out, typename T, typename Pred, typename Op,
          typename = typename std::enable_if<!detail::is_execution_policy<KIt>::value>::type>
Out exclusive_scan_by_key(KIt kf, KIt kl, VIt vf, Out result, T init, Pred pred, Op op) {
  return thrust::exclusive_scan_by_key(detail::policy_for<KIt>(), kf, kl, vf, result, init, pred, op);
}

}  // namespace thrust

#if defined(__HIPCC__)
#include <thrust/system/hip/detail/generic_by_key.h>
#endif
