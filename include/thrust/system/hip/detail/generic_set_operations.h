// set_difference, set_intersection, set_symmetric_difference, set_union and their _by_key
// forms for a user's comparator or key struct (hipcc translation units).
//
// For a key x with m equivalents in A and n in B, the reference's sequential loop
// (thrust/system/detail/sequential/set_operations.h:42-215) keeps
//   difference            A_r with r >= n
//   intersection          A_r with r <  n
//   symmetric difference  A_r with r >= n and B_r with r >= m
//   union                 every A_r     and B_r with r >= m
// in the order of the stable merge (A first among equivalents).  Every element decides for
// itself, with binary searches in the two sorted ranges:
//   A_r  sits at merged position (own index) + (elements of B before x); it has a partner
//        when the element r places past B's first "not before x" is equivalent to x
//   B_r  sits at (own index) + (elements of A not after x); it has a partner when the
//        element r + 1 places before A's first "after x" is equivalent to x
// One kernel, instantiated for the comparator, writes keys (and values) to their merged
// positions with a keep byte each (a workgroup takes a chunk of one range, whose ends bound
// the chunk's searches in the other range); the library's compaction kernel, with those bytes as
// its stencil, writes the result.  Keys and values are moved as items of 1, 2, 4 or 8 bytes.
#pragma once
#if !defined(__HIPCC__)
#error "thrust/system/hip/detail/generic_set_operations.h is HIP code: compile this translation unit with hipcc"
#endif
#include <thrust/pair.h>
#include <thrust/system/hip/detail/device_input.h>
#include <thrust/system/hip/detail/generic_by_key.h>

namespace thrust {
namespace system {
namespace hip {
namespace detail {

// first index in [lo, hi) whose element is not before x
template <typename K, typename Comp>
__device__ __forceinline__ uint64_t set_lower_bound(const K* p, uint64_t lo, uint64_t hi, const K& x, Comp& comp) {
  while (lo < hi) {
    const uint64_t mid = lo + ((hi - lo) >> 1);
    if (comp(p[mid], x)) lo = mid + 1;
    else hi = mid;
  }
  return lo;
}
// first index in [lo, hi) whose element is after x
template <typename K, typename Comp>
__device__ __forceinline__ uint64_t set_upper_bound(const K* p, uint64_t lo, uint64_t hi, const K& x, Comp& comp) {
  while (lo < hi) {
    const uint64_t mid = lo + ((hi - lo) >> 1);
    if (!comp(x, p[mid])) lo = mid + 1;
    else hi = mid;
  }
  return lo;
}
// rank of p[i] among its equivalents in the sorted range p: runs are short as a rule, so the
// search gallops back from i before it bisects
template <typename K, typename Comp>
__device__ __forceinline__ uint64_t set_rank_in_run(const K* p, uint64_t i, const K& x, Comp& comp) {
  uint64_t hi = i, step = 1;  // p[hi] is equivalent to x
  while (hi >= step && !comp(p[hi - step], x)) {
    hi -= step;
    step <<= 1;
  }
  const uint64_t lo = hi >= step ? hi - step + 1 : 0;  // p[lo - 1] is before x, or lo == 0
  return i - set_lower_bound(p, lo, hi, x, comp);
}

// a = both, b = both + na.  merged[p], merged_values[p], keep[p] for the merged position p of
// every element of the two ranges.  A workgroup takes SET_CHUNK consecutive elements of one
// range; the places of the chunk's first and last element in the other range bound every
// search of the chunk there, so only two searches per workgroup run over the whole range.
constexpr int SET_CHUNK = ELEMENTWISE_BLOCK * 8;
template <typename K, typename V, bool HAS_VALUES, typename Comp>
__global__ __launch_bounds__(ELEMENTWISE_BLOCK) void set_place_kernel(const K* both, const V* both_values, uint64_t na,
                                                                      uint64_t nb, uint64_t chunks_a, int op, Comp comp,
                                                                      K* merged, V* merged_values, unsigned char* keep) {
  __shared__ uint64_t s_bound[2];
  const K* a = both;
  const K* b = both + na;
  const bool a_alone = op != THRUST_AMD_SET_INTERSECTION;                                  // A without partner
  const bool a_paired = op == THRUST_AMD_SET_INTERSECTION || op == THRUST_AMD_SET_UNION;  // A with partner
  const bool b_alone = op == THRUST_AMD_SET_SYMMETRIC_DIFFERENCE || op == THRUST_AMD_SET_UNION;
  const bool from_a = blockIdx.x < chunks_a;
  const K* own = from_a ? a : b;
  const K* other = from_a ? b : a;
  const uint64_t n_own = from_a ? na : nb, n_other = from_a ? nb : na;
  const uint64_t begin = (from_a ? (uint64_t)blockIdx.x : (uint64_t)blockIdx.x - chunks_a) * SET_CHUNK;
  const uint64_t end = begin + SET_CHUNK < n_own ? begin + SET_CHUNK : n_own;
  // elements of the other range before the chunk's first key / not after its last key
  if (threadIdx.x == 0) s_bound[0] = set_lower_bound(other, (uint64_t)0, n_other, own[begin], comp);
  if (threadIdx.x == 64) s_bound[1] = set_upper_bound(other, (uint64_t)0, n_other, own[end - 1], comp);
  __syncthreads();
  const uint64_t lo = s_bound[0], hi = s_bound[1];
  for (uint64_t i = begin + threadIdx.x; i < end; i += ELEMENTWISE_BLOCK) {
    const K x = own[i];
    const uint64_t r = set_rank_in_run(own, i, x, comp);
    uint64_t at;
    bool kept;
    if (from_a) {
      const uint64_t before = set_lower_bound(b, lo, hi, x, comp);
      const bool partner = before + r < nb && !comp(x, b[before + r]);
      at = i + before;
      kept = partner ? a_paired : a_alone;
    } else {
      const uint64_t upto = set_upper_bound(a, lo, hi, x, comp);
      const bool partner = r < upto && !comp(a[upto - 1 - r], x);
      at = i + upto;
      kept = b_alone && !partner;
    }
    merged[at] = x;
    if (HAS_VALUES) merged_values[at] = both_values[(from_a ? 0 : na) + i];
    keep[at] = kept ? 1 : 0;
  }
}

// vf2 is not read when the operation never keeps an element of the second range.
template <int OP, typename D, typename K1, typename K2, typename V1, typename V2, typename KOut, typename VOut,
          typename Comp>
uint64_t set_operation_generic(execution_policy<D>& exec, K1 kf1, K1 kl1, K2 kf2, K2 kl2, V1 vf1, V2 vf2, KOut ko,
                               VOut vo, Comp comp, bool has_values) {
  typedef typename std::remove_const<typename iterator_value<K1>::type>::type K;
  typedef typename iterator_value<VOut>::type V;
  static_assert(is_abi_item<K>::value && std::is_same<typename iterator_value<KOut>::type, K>::value &&
                    std::is_same<typename std::remove_const<typename iterator_value<K2>::type>::type, K>::value,
                "set operations on the device system: keys of 1, 2, 4 or 8 bytes, one type for both inputs and the output");
  static_assert(is_abi_item<V>::value, "set operations by key on the device system: values of 1, 2, 4 or 8 bytes");
  void* stream = stream_of(exec);
  const uint64_t na = (uint64_t)(kl1 - kf1), nb = (uint64_t)(kl2 - kf2), n = na + nb;
  if (n == 0) return 0;
  const bool keeps_second = OP == THRUST_AMD_SET_SYMMETRIC_DIFFERENCE || OP == THRUST_AMD_SET_UNION;
  const std::size_t key_bytes = ((std::size_t)n * sizeof(K) + 255) / 256 * 256;
  const std::size_t val_bytes = has_values ? ((std::size_t)n * sizeof(V) + 255) / 256 * 256 : 0;
  temp_storage temp(stream, temp_source_of(exec));
  temp.ensure(2 * (key_bytes + val_bytes) + (std::size_t)n);
  char* base = static_cast<char*>(temp.ptr());
  K* both = reinterpret_cast<K*>(base);
  K* merged = reinterpret_cast<K*>(base + key_bytes);
  V* both_values = reinterpret_cast<V*>(base + 2 * key_bytes);
  V* merged_values = reinterpret_cast<V*>(base + 2 * key_bytes + val_bytes);
  unsigned char* keep = reinterpret_cast<unsigned char*>(base + 2 * (key_bytes + val_bytes));
  materialize(stream, kf1, both, na);
  materialize(stream, kf2, both + na, nb);
  const uint64_t chunks_a = (na + SET_CHUNK - 1) / SET_CHUNK, chunks_b = (nb + SET_CHUNK - 1) / SET_CHUNK;
  if (chunks_a + chunks_b > 0x7fffffffull) throw_on_error(1, "set operation: ranges too long");
  if (has_values) {
    materialize(stream, vf1, both_values, na);
    if (keeps_second) materialize(stream, vf2, both_values + na, nb);
    hipLaunchKernelGGL((set_place_kernel<K, V, true, Comp>), dim3((unsigned)(chunks_a + chunks_b)),
                       dim3(ELEMENTWISE_BLOCK), 0, (hipStream_t)stream, (const K*)both, (const V*)both_values, na, nb,
                       chunks_a, (int)OP, comp, merged, merged_values, keep);
  } else {
    hipLaunchKernelGGL((set_place_kernel<K, V, false, Comp>), dim3((unsigned)(chunks_a + chunks_b)),
                       dim3(ELEMENTWISE_BLOCK), 0, (hipStream_t)stream, (const K*)both, (const V*)nullptr, na, nb,
                       chunks_a, (int)OP, comp, merged, (V*)nullptr, keep);
  }
  throw_on_error(launch_status(), "set operation: kernel launch");
  const uint64_t cnt = select_by_flags(stream, temp_source_of(exec), merged, keep, thrust::detail::raw(ko), n, sizeof(K),
                                       "set operation failed");
  if (has_values)
    (void)select_by_flags(stream, temp_source_of(exec), merged_values, keep, thrust::detail::raw(vo), n, sizeof(V),
                          "set operation by key failed");
  return cnt;
}

}  // namespace detail
}  // namespace hip
}  // namespace system
}  // namespace thrust
