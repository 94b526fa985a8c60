// unique, unique_by_key, reduce_by_key and scan_by_key for a user's key predicate, operator or
// element structs (hipcc translation units).
//
//   unique, unique_by_key   the single-pass compaction kernel, instantiated for the predicate
//                           (thrust/system/hip/detail/generic_select.h)
//   reduce_by_key           the single-pass segmented reduction, instantiated for the predicate and
//                           the operator (thrust/system/hip/detail/reduce_by_key_kernels.h), when
//                           the sums have the values' own type and keys and values are items of
//                           up to 8 bytes
//   scan_by_key             the single-pass segmented scan (thrust/system/hip/detail/scan_by_key_kernels.h)
//                           under the same conditions, written to device memory
//   otherwise a composition of pieces:
//     run flags   one kernel, instantiated for the predicate: head[i] = i == 0 || !pred(k[i-1], k[i])
//                 and tail[i] = i == n-1 || !pred(k[i], k[i+1]), one byte each
//                 (thrust/detail/range/head_flags.h:130-160, tail_flags.h in the reference)
//     sums        (head, value) pairs scanned with the segmented form of the operator through
//                 the generic in-order scan, the reference's formulation
//                 (thrust/system/detail/generic/reduce_by_key.inl:50-136); the pairs are made as
//                 the scan reads them and only the values are written; the value at a run's
//                 tail is the run's sum
//     selection   the library's compaction kernel with the flag bytes as its stencil: the keys at
//                 the heads, the sums at the tails
#pragma once
#if !defined(__HIPCC__)
#error "thrust/system/hip/detail/generic_by_key.h is HIP code: compile this translation unit with hipcc"
#endif
#include <thrust/copy.h>
#include <thrust/iterator/counting_iterator.h>
#include <thrust/iterator/transform_iterator.h>
#include <thrust/pair.h>
#include <thrust/scan.h>
#include <thrust/system/hip/detail/device_input.h>
#include <thrust/system/hip/detail/generic_select.h>
#include <thrust/system/hip/detail/reduce_by_key_kernels.h>
#include <thrust/system/hip/detail/scan_by_key_kernels.h>

namespace thrust {
namespace system {
namespace hip {
namespace detail {

template <typename ViewK, typename Pred>
__global__ __launch_bounds__(ELEMENTWISE_BLOCK) void run_flags_kernel(ViewK keys, uint64_t n, Pred pred,
                                                                      unsigned char* head, unsigned char* tail) {
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    head[i] = (i == 0 || !pred(keys[i - 1], keys[i])) ? 1 : 0;
    if (tail) tail[i] = (i == n - 1 || !pred(keys[i], keys[i + 1])) ? 1 : 0;
  }
}

template <typename V>
struct seg_pair {
  V value;
  unsigned char head;
  // a scan over pairs may write the values alone
  __host__ __device__ explicit operator V() const { return value; }
};
// element i of the (head, value) pairs of a segmented scan, made as it is read
template <typename ViewV, typename V>
struct seg_pair_at {
  ViewV values;
  const unsigned char* head;
  __host__ __device__ seg_pair<V> operator()(uint64_t i) const {
    seg_pair<V> p;
    p.value = (V)values[i];
    p.head = head[i];
    return p;
  }
};
template <typename V, typename Op>
struct seg_op {  // the operator of a segmented scan: a head on the right starts over
  Op op;
  __host__ __device__ seg_pair<V> operator()(const seg_pair<V>& a, const seg_pair<V>& b) const {
    seg_pair<V> r;
    r.head = (unsigned char)(a.head | b.head);
    r.value = b.head ? b.value : (V)op(a.value, b.value);
    return r;
  }
};
template <typename V>
struct pair_value {
  __host__ __device__ V operator()(const seg_pair<V>& p) const { return p.value; }
};
template <typename ViewV, typename V>
__global__ __launch_bounds__(ELEMENTWISE_BLOCK) void seg_pairs_kernel(ViewV values, const unsigned char* head,
                                                                      uint64_t n, seg_pair<V>* pairs) {
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    seg_pair<V> p;
    p.value = (V)values[i];
    p.head = head[i];
    pairs[i] = p;
  }
}

// items[i] with flags[i] != 0, compacted in order into out; returns how many.
inline uint64_t select_by_flags(void* stream, const temp_source& source, const void* items, const unsigned char* flags,
                                void* out, uint64_t n, std::size_t item_bytes, const char* what) {
  return run_selection<unsigned char>(
      stream, source, thrust::identity<unsigned char>(), what,
      [&](void* t, std::size_t* b, uint64_t* d_num, int cmp, const void* thr) {
        return thrust_amd_copy_if(t, b, items, flags, out, d_num, n, item_bytes, THRUST_AMD_U8, cmp, thr, stream);
      });
}

template <typename D, typename KIn, typename Pred>
inline void launch_run_flags(execution_policy<D>& exec, KIn kf, uint64_t n, Pred pred, unsigned char* head,
                             unsigned char* tail) {
  typedef typename thrust::detail::device_view_of<KIn>::type View;
  hipLaunchKernelGGL((run_flags_kernel<View, Pred>), dim3(elementwise_grid(n)), dim3(ELEMENTWISE_BLOCK), 0,
                     (hipStream_t)stream_of(exec), thrust::detail::device_view(kf), n, pred, head, tail);
  throw_on_error(launch_status(), "run flags: kernel launch");
}

template <typename D, typename In, typename Out, typename Pred>
Out unique_copy_generic(execution_policy<D>& exec, In first, In last, Out result, Pred pred) {
  typedef typename std::remove_const<typename iterator_value<In>::type>::type T;
  static_assert(is_abi_item<T>::value && std::is_same<typename iterator_value<Out>::type, T>::value,
                "unique on the device system: items of 1, 2, 4 or 8 bytes, same type in and out");
  void* stream = stream_of(exec);
  const uint64_t n = (uint64_t)(last - first);
  if (n == 0) return result;
  device_input<In> source(stream, temp_source_of(exec), first, n);
  const uint64_t cnt = generic_unique(stream, temp_source_of(exec), (const T*)source.ptr(), thrust::detail::raw(result),
                                      n, pred, "unique failed");
  return result + cnt;
}

template <typename D, typename KIn, typename VIn, typename KOut, typename VOut, typename Pred>
pair<KOut, VOut> unique_by_key_copy_generic(execution_policy<D>& exec, KIn kf, KIn kl, VIn vf, KOut ko, VOut vo,
                                            Pred pred) {
  typedef typename std::remove_const<typename iterator_value<KIn>::type>::type K;
  typedef typename std::remove_const<typename iterator_value<VIn>::type>::type V;
  static_assert(is_abi_item<K>::value && std::is_same<typename iterator_value<KOut>::type, K>::value &&
                    is_abi_item<V>::value && std::is_same<typename iterator_value<VOut>::type, V>::value,
                "unique_by_key on the device system: keys and values of 1, 2, 4 or 8 bytes, same types in and out");
  void* stream = stream_of(exec);
  const uint64_t n = (uint64_t)(kl - kf);
  if (n == 0) return thrust::make_pair(ko, vo);
  device_input<KIn> keys(stream, temp_source_of(exec), kf, n);
  device_input<VIn> values(stream, temp_source_of(exec), vf, n);
  const uint64_t cnt = generic_unique_by_key(stream, temp_source_of(exec), (const K*)keys.ptr(), (const V*)values.ptr(),
                                             thrust::detail::raw(ko), thrust::detail::raw(vo), n, pred,
                                             "unique_by_key failed");
  return thrust::make_pair(ko + cnt, vo + cnt);
}

// Keys and values the single-pass kernel takes as they are: keys of up to 8 bytes, values of the
// output's own type, 4 or 8 bytes wide (or a narrow integer, which travels widened).
template <typename K, typename VI, typename V>
struct reduces_by_key_in_one_pass
    : std::integral_constant<bool, is_kernel_item<K>::value && sizeof(K) <= 8 && std::is_same<VI, V>::value &&
                                       is_kernel_item<V>::value &&
                                       (sizeof(V) == 4 || sizeof(V) == 8 || std::is_same<V, int8_t>::value ||
                                        std::is_same<V, uint8_t>::value || std::is_same<V, int16_t>::value ||
                                        std::is_same<V, uint16_t>::value)> {};

// The single-pass kernel, instantiated for the caller's key equality and operator.
template <typename D, typename KIn, typename VIn, typename KOut, typename VOut, typename Pred, typename Op>
pair<KOut, VOut> reduce_by_key_one_pass(execution_policy<D>& exec, KIn kf, KIn kl, VIn vf, KOut ko, VOut vo, Pred pred,
                                        Op op) {
  namespace seg = ::thrust::system::hip::segmented;
  typedef typename std::remove_const<typename iterator_value<KIn>::type>::type K;
  typedef typename iterator_value<VOut>::type V;
  void* stream = stream_of(exec);
  const uint64_t n = (uint64_t)(kl - kf);
  device_input<KIn> keys(stream, temp_source_of(exec), kf, n);
  device_input<VIn> values(stream, temp_source_of(exec), vf, n);
  const seg::RbkTemp<K, V> lay(n);
  temp_storage temp(stream, temp_source_of(exec));
  temp.ensure(lay.total + 256);
  char* base = static_cast<char*>(temp.ptr());
  uint64_t* d_num = reinterpret_cast<uint64_t*>(base + lay.total);
  seg::RbkArgs<K, V, Pred, Op> a = seg::make_rbk_args<K, V>(pred, op);
  a.keys = (const K*)keys.ptr();
  a.values = (const V*)values.ptr();
  a.keys_out = thrust::detail::raw(ko);
  a.values_out = thrust::detail::raw(vo);
  a.d_num_runs = d_num;
  a.n = n;
  throw_on_error(seg::rbk_launch(base, a, (hipStream_t)stream), "reduce_by_key failed");
  const uint64_t runs = read_scalar<uint64_t>(d_num, stream, "reduce_by_key failed");
  return thrust::make_pair(ko + runs, vo + runs);
}

template <typename D, typename KIn, typename VIn, typename KOut, typename VOut, typename Pred, typename Op>
pair<KOut, VOut> reduce_by_key_generic(execution_policy<D>& exec, KIn kf, KIn kl, VIn vf, KOut ko, VOut vo, Pred pred,
                                       Op op) {
  typedef typename std::remove_const<typename iterator_value<KIn>::type>::type K;
  typedef typename iterator_value<VOut>::type V;  // sums have the output's value type
  typedef typename std::remove_const<typename iterator_value<VIn>::type>::type VI;
  if constexpr (reduces_by_key_in_one_pass<K, VI, V>::value && std::is_same<typename iterator_value<KOut>::type, K>::value) {
    // the kernel counts runs in 32 bits; beyond that the composition below takes over
    if ((uint64_t)(kl - kf) < 0xffffffffull) return reduce_by_key_one_pass(exec, kf, kl, vf, ko, vo, pred, op);
  }
  static_assert(is_abi_item<K>::value && std::is_same<typename iterator_value<KOut>::type, K>::value &&
                    is_abi_item<V>::value,
                "reduce_by_key on the device system: keys and sums of 1, 2, 4 or 8 bytes, same key type in and out");
  void* stream = stream_of(exec);
  const uint64_t n = (uint64_t)(kl - kf);
  if (n == 0) return thrust::make_pair(ko, vo);
  device_input<KIn> keys(stream, temp_source_of(exec), kf, n);
  temp_storage flags(stream, temp_source_of(exec));
  flags.ensure((std::size_t)n * 2);
  unsigned char* head = static_cast<unsigned char*>(flags.ptr());
  unsigned char* tail = head + n;
  launch_run_flags(exec, keys.ptr(), n, pred, head, tail);

  // the running sums of the runs: the generic in-order scan reads (head, value) pairs made on
  // the fly and writes the values alone
  typedef seg_pair<V> P;
  typedef typename thrust::detail::device_view_of<VIn>::type ViewV;
  temp_storage sum_store(stream, temp_source_of(exec));
  sum_store.ensure((std::size_t)n * sizeof(V));
  V* sums = static_cast<V*>(sum_store.ptr());
  const seg_pair_at<ViewV, V> pair_at = {thrust::detail::device_view(vf), head};
  const seg_op<V, Op> sop = {op};
  scan_generic<false, P>(exec, thrust::make_transform_iterator(thrust::counting_iterator<uint64_t>(0), pair_at),
                         thrust::make_transform_iterator(thrust::counting_iterator<uint64_t>(n), pair_at), sums, P(), sop);
  const uint64_t runs = select_by_flags(stream, temp_source_of(exec), sums, tail, thrust::detail::raw(vo), n,
                                        sizeof(V), "reduce_by_key failed");
  (void)select_by_flags(stream, temp_source_of(exec), keys.ptr(), head, thrust::detail::raw(ko), n, sizeof(K),
                        "reduce_by_key failed");
  return thrust::make_pair(ko + runs, vo + runs);
}

// inclusive / exclusive scan_by_key: the generic in-order scan over (head, value) pairs with the
// segmented operator.  The exclusive form scans the values shifted right by one with init at
// the heads, which is how the reference states it
// (thrust/system/detail/generic/scan_by_key.inl:50-140).  A is the accumulator's type.
template <typename ViewV, typename A>
__global__ __launch_bounds__(ELEMENTWISE_BLOCK) void shifted_seg_pairs_kernel(ViewV values, const unsigned char* head,
                                                                              uint64_t n, A init, seg_pair<A>* pairs) {
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    seg_pair<A> p;
    p.head = head[i];
    if (p.head) p.value = init;
    else p.value = (A)values[i - 1];
    pairs[i] = p;
  }
}

// The single-pass segmented scan, instantiated for the caller's key equality and operator: keys of
// up to 8 bytes, values, accumulator and output of one type (4 or 8 bytes, or a narrow integer),
// written to device memory.
template <typename K, typename VI, typename A, typename Out>
struct scans_by_key_in_one_pass
    : std::integral_constant<bool, reduces_by_key_in_one_pass<K, VI, A>::value &&
                                       std::is_same<typename iterator_value<Out>::type, A>::value &&
                                       (std::is_pointer<Out>::value || thrust::detail::is_device_iterator<Out>::value)> {};
template <bool EXCLUSIVE, typename D, typename KIt, typename VIt, typename Out, typename A, typename Pred, typename Op>
Out scan_by_key_one_pass(execution_policy<D>& exec, KIt kf, KIt kl, VIt vf, Out result, A init, Pred pred, Op op) {
  namespace seg = ::thrust::system::hip::segmented;
  typedef typename std::remove_const<typename iterator_value<KIt>::type>::type K;
  void* stream = stream_of(exec);
  const uint64_t n = (uint64_t)(kl - kf);
  device_input<KIt> keys(stream, temp_source_of(exec), kf, n);
  device_input<VIt> values(stream, temp_source_of(exec), vf, n);
  const A* in = (const A*)values.ptr();
  A* out = (A*)thrust::detail::raw(result);  // either form may write onto its values
  const seg::SbkTemp<K, A> lay(n);
  temp_storage temp(stream, temp_source_of(exec));
  temp.ensure(lay.total);
  throw_on_error(seg::sbk_launch(static_cast<char*>(temp.ptr()), (const K*)keys.ptr(), in, out, n, EXCLUSIVE, init, pred, op,
                                 (hipStream_t)stream),
                 "scan_by_key failed");
  synchronize(stream, "scan_by_key: synchronize");
  return result + n;
}

template <bool EXCLUSIVE, typename D, typename KIt, typename VIt, typename Out, typename A, typename Pred, typename Op>
Out scan_by_key_generic(execution_policy<D>& exec, KIt kf, KIt kl, VIt vf, Out result, A init, Pred pred, Op op) {
  static_assert(is_device_input<KIt>::value && is_device_input<VIt>::value && is_device_output<Out>::value,
                "scan_by_key on the device system reads device or fancy iterators and writes device memory");
  void* stream = stream_of(exec);
  const uint64_t n = (uint64_t)(kl - kf);
  if (n == 0) return result;
  {
    typedef typename std::remove_const<typename iterator_value<KIt>::type>::type K;
    typedef typename std::remove_const<typename iterator_value<VIt>::type>::type VI;
    if constexpr (scans_by_key_in_one_pass<K, VI, A, Out>::value) {
      // the kernel counts run beginnings in 32 bits; beyond that the composition below takes over
      if (n < 0xffffffffull) return scan_by_key_one_pass<EXCLUSIVE>(exec, kf, kl, vf, result, init, pred, op);
    }
  }
  temp_storage flags(stream, temp_source_of(exec));
  flags.ensure((std::size_t)n);
  unsigned char* head = static_cast<unsigned char*>(flags.ptr());
  launch_run_flags(exec, kf, n, pred, head, nullptr);
  typedef seg_pair<A> P;
  typedef typename thrust::detail::device_view_of<VIt>::type ViewV;
  const seg_op<A, Op> sop = {op};
  constexpr bool writes_values = !EXCLUSIVE &&
                                 (std::is_pointer<Out>::value || thrust::detail::is_device_iterator<Out>::value) &&
                                 std::is_same<typename iterator_value<Out>::type, A>::value;
  if constexpr (writes_values) {
    // inclusive: the pairs are made as the scan reads them and the values alone are written.
    // The output may be the input: a tile is read completely before any of it is written,
    // and no tile reads another tile's elements.
    const seg_pair_at<ViewV, A> pair_at = {thrust::detail::device_view(vf), head};
    scan_generic<false, P>(exec, thrust::make_transform_iterator(thrust::counting_iterator<uint64_t>(0), pair_at),
                           thrust::make_transform_iterator(thrust::counting_iterator<uint64_t>(n), pair_at),
                           thrust::detail::raw(result), P(), sop);
    return result + n;
  }
  // exclusive: element i takes the value of element i - 1, which may lie in another tile, so
  // the pairs are written out first
  temp_storage pair_store(stream, temp_source_of(exec));
  pair_store.ensure((std::size_t)n * sizeof(P));
  P* pairs = static_cast<P*>(pair_store.ptr());
  if (EXCLUSIVE)
    hipLaunchKernelGGL((shifted_seg_pairs_kernel<ViewV, A>), dim3(elementwise_grid(n)), dim3(ELEMENTWISE_BLOCK), 0,
                       (hipStream_t)stream, thrust::detail::device_view(vf), (const unsigned char*)head, n, init, pairs);
  else
    hipLaunchKernelGGL((seg_pairs_kernel<ViewV, A>), dim3(elementwise_grid(n)), dim3(ELEMENTWISE_BLOCK), 0,
                       (hipStream_t)stream, thrust::detail::device_view(vf), (const unsigned char*)head, n, pairs);
  throw_on_error(launch_status(), "scan_by_key: kernel launch");
  scan_generic<false, P>(exec, pairs, pairs + n, pairs, P(), sop);
  // the values of the scanned pairs are the result (the pairs were built from a copy of the
  // input, so the output may be the input)
  materialize(stream, thrust::make_transform_iterator((const P*)pairs, pair_value<A>()), result, n);
  synchronize(stream, "scan_by_key: synchronize");
  return result + n;
}

}  // namespace detail
}  // namespace hip
}  // namespace system
}  // namespace thrust
