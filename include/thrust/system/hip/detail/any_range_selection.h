// Selection (copy_if, remove_copy_if, partition_copy, stable_partition, with or without
// stencil) for ranges the compaction kernels do not take: elements of any size (a zip of
// arrays, a struct), inputs and outputs that are not arrays in memory (zip iterators,
// discard_iterator, a caller's own iterator type), outputs of another element type.  The
// reference's agents read and write through the iterators themselves
// (thrust/system/cuda/detail/copy_if.h:365-478, partition.h:221-293); here such ranges take
// three passes instead of one:
//   1. the predicate of element i (or of stencil[i]) as a 32-bit 0 / 1, by the kernel that
//      materialises any iterator;
//   2. an inclusive scan of those words in place (the library's scan): word i is then the
//      number of selected elements up to and including i;
//   3. one thread per element writes in[i] to out_true[count - 1] or out_false[i - count]
//      through the iterators.
// The input is copied into temporary storage first, so a range may be partitioned onto
// itself.  HBM traffic: the element read three times and written twice, 12 bytes of
// counts per element.  Needs hipcc (the kernels are templates on the iterators).
#pragma once
#if !defined(__HIPCC__)
#error "thrust/system/hip/detail/any_range_selection.h is HIP code: compile this translation unit with hipcc"
#endif
#include <thrust/iterator/discard_iterator.h>
#include <thrust/iterator/transform_iterator.h>
#include <thrust/system/hip/detail/device_input.h>

namespace thrust {
namespace system {
namespace hip {
namespace detail {

template <typename Pred>
struct as_count {
  mutable Pred pred;  // a caller's predicate need not be const-callable
  bool negate;
  template <typename V>
  __host__ __device__ uint32_t operator()(const V& x) const { return ((pred(x) ? true : false) != negate) ? 1u : 0u; }
};

template <typename T, typename OutTrue, typename OutFalse, bool HAS_FALSE>
__global__ __launch_bounds__(ELEMENTWISE_BLOCK) void scatter_by_count_kernel(const T* in, const uint32_t* counts,
                                                                             OutTrue out_true, OutFalse out_false,
                                                                             uint64_t n) {
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    const uint32_t upto = counts[i];
    const uint32_t before = i ? counts[i - 1] : 0u;
    if (upto != before) out_true[upto - 1] = in[i];
    else if (HAS_FALSE) out_false[i - upto] = in[i];
  }
}

// Steps 1 and 2: the input copied into `items`, the running counts in `counts`; returns the
// number of selected elements (pred(stencil[i]) != negate).
template <typename D, typename In, typename St, typename Pred>
inline uint64_t count_any_range(execution_policy<D>& exec, In first, uint64_t n, St stencil, Pred pred, bool negate,
                                temp_storage& items, temp_storage& count_store, const char* what) {
  typedef typename std::remove_const<typename iterator_value<In>::type>::type T;
  static_assert(is_bytewise_movable<T>::value, "selection on the device system: elements are moved as bytes");
  if (n >= 0xffffffffull) throw thrust::system::system_error((int)hipErrorInvalidValue, what);  // 32-bit counts
  void* stream = stream_of(exec);
  items.ensure((std::size_t)n * sizeof(T));
  materialize(stream, first, static_cast<T*>(items.ptr()), n);
  count_store.ensure((std::size_t)n * sizeof(uint32_t));
  uint32_t* counts = static_cast<uint32_t*>(count_store.ptr());
  materialize(stream, thrust::make_transform_iterator(stencil, as_count<Pred>{pred, negate}), counts, n);
  temp_storage temp(stream, temp_source_of(exec));
  (void)run(temp, 0, what, [&](void* t, std::size_t* b) {
    return thrust_amd_inclusive_scan(t, b, counts, counts, n, THRUST_AMD_U32, THRUST_AMD_PLUS, stream);
  });
  return read_scalar<uint32_t>(counts + (n - 1), stream, what);
}

// Step 3.
template <bool HAS_FALSE, typename T, typename OutTrue, typename OutFalse>
inline void scatter_any_range(void* stream, const temp_storage& items, const temp_storage& count_store, uint64_t n,
                              OutTrue out_true, OutFalse out_false, const char* what) {
  typedef typename thrust::detail::device_view_of<OutTrue>::type ViewTrue;
  typedef typename thrust::detail::device_view_of<OutFalse>::type ViewFalse;
  hipLaunchKernelGGL((scatter_by_count_kernel<T, ViewTrue, ViewFalse, HAS_FALSE>), dim3(elementwise_grid(n)),
                     dim3(ELEMENTWISE_BLOCK), 0, (hipStream_t)stream, static_cast<const T*>(items.ptr()),
                     static_cast<const uint32_t*>(count_store.ptr()), thrust::detail::device_view(out_true),
                     thrust::detail::device_view(out_false), n);
  throw_on_error(launch_status(), what);
  synchronize(stream, what);  // the temporaries go back to the arena when the caller returns
}

// Selected elements to out_true[0, count), the others to out_false[0, n - count) when
// HAS_FALSE; returns count.  The outputs may overlap the input.
template <bool HAS_FALSE, typename D, typename In, typename St, typename OutTrue, typename OutFalse, typename Pred>
inline uint64_t select_any_range(execution_policy<D>& exec, In first, uint64_t n, St stencil, OutTrue out_true,
                                 OutFalse out_false, Pred pred, bool negate, const char* what) {
  typedef typename std::remove_const<typename iterator_value<In>::type>::type T;
  if (n == 0) return 0;
  temp_storage items(stream_of(exec), temp_source_of(exec)), counts(stream_of(exec), temp_source_of(exec));
  const uint64_t count = count_any_range(exec, first, n, stencil, pred, negate, items, counts, what);
  scatter_any_range<HAS_FALSE, T>(stream_of(exec), items, counts, n, out_true, out_false, what);
  return count;
}

// The range partitioned onto itself: selected elements first, the others behind them, both in
// their order; returns the number selected.
template <typename D, typename It, typename St, typename Pred>
inline uint64_t partition_any_range(execution_policy<D>& exec, It first, uint64_t n, St stencil, Pred pred,
                                    const char* what) {
  typedef typename std::remove_const<typename iterator_value<It>::type>::type T;
  if (n == 0) return 0;
  temp_storage items(stream_of(exec), temp_source_of(exec)), counts(stream_of(exec), temp_source_of(exec));
  const uint64_t count = count_any_range(exec, first, n, stencil, pred, false, items, counts, what);
  scatter_any_range<true, T>(stream_of(exec), items, counts, n, first, first + count, what);
  return count;
}

}  // namespace detail
}  // namespace hip
}  // namespace system
}  // namespace thrust
