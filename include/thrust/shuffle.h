// thrust::shuffle, thrust::shuffle_copy: a random permutation of a range, drawn from a caller's
// uniform random bit generator (thrust/shuffle.h:60-180; thrust/system/detail/generic/shuffle.inl:
// 30-190; testing/shuffle.cu).
//
// The permutation is the reference's, bit for bit: sixteen draws of the generator key a Feistel
// network over the next power of two n >= m, element i of the output is the input at the i-th
// of the images b(0), b(1), ... b(n-1) that fall below m.  Here the images are computed once
// into a buffer of n 64-bit keys (one transform), and one stream compaction gathers through the
// keys it keeps: 8 n bytes written and read beside the data, where the reference folds both
// into a scan with a side-effecting output iterator.
#pragma once
#include <cstddef>
#include <cstdint>

#include <thrust/copy.h>
#include <thrust/device_vector.h>
#include <thrust/host_vector.h>
#include <thrust/iterator/counting_iterator.h>
#include <thrust/iterator/transform_iterator.h>
#include <thrust/random.h>
#include <thrust/system/hip/detail/backend.h>
#include <thrust/transform.h>

namespace thrust {

template <typename D, typename It, typename Out, typename URBG>
void shuffle_copy(const detail::execution_policy_base<D>& exec, It first, It last, Out result, URBG&& g);

namespace detail {
// The keyed permutation of [0, 2^w), w = bits needed for m - 1, that the reference draws its shuffle
// from (generic/shuffle.inl:34-140 states the arithmetic; tests/golden/shuffle_permutations.npz pins
// it).  An index is split into a high part of floor(w / 2) bits and a low part of the remaining
// bits.  Sixteen times over, the low part's narrow bits move up to become the high part, and the old
// high part, xor-ed with a keyed hash of the whole low part, moves down; when w is odd the low
// part's extra top bit stays at the bottom of the new low part.  The sixteen keys are the first
// sixteen draws of the caller's generator.
struct index_cipher {
  std::uint64_t round_key[16];
  unsigned narrow;  // bits of the high part
  unsigned wide;    // bits of the low part: narrow, or narrow + 1
};

template <typename URBG>
__host__ __device__ index_cipher make_index_cipher(std::uint64_t m, URBG&& g) {
  unsigned w = 0;
  for (std::uint64_t top = m > 0 ? m - 1 : 0; top != 0; top >>= 1) ++w;
  index_cipher c;
  c.narrow = w / 2;
  c.wide = w - c.narrow;
  for (std::uint64_t& k : c.round_key) k = g();
  return c;
}

__host__ __device__ inline std::uint64_t cipher_domain(const index_cipher& c) { return 1ull << (c.narrow + c.wide); }

// a ^= b + golden ratio + (a << 6) + (a >> 2): how the round function folds its three ingredients
__host__ __device__ inline std::uint64_t fold_into(std::uint64_t a, std::uint64_t b) {
  return a ^ (b + 0x9e3779b9 + (a << 6) + (a >> 2));
}

__host__ __device__ inline std::uint64_t encipher(const index_cipher& c, std::uint64_t index) {
  const std::uint32_t narrow_mask = static_cast<std::uint32_t>((1ull << c.narrow) - 1);
  std::uint32_t hi = static_cast<std::uint32_t>(index >> c.wide);
  std::uint32_t lo = static_cast<std::uint32_t>(index & ((1ull << c.wide) - 1));
  for (const std::uint64_t key : c.round_key) {
    // the first draw of a taus88 seeded with the low part, the round's key, and the first draw of
    // a ranlux48 seeded with the low part
    const std::uint64_t from_taus = thrust::random::taus88(lo)();
    const std::uint64_t from_ranlux = thrust::random::ranlux48(static_cast<std::uint64_t>(lo))();
    const std::uint32_t mask = static_cast<std::uint32_t>(fold_into(fold_into(from_taus, key), from_ranlux)) & narrow_mask;
    // (lo >> narrow is the extra top bit of an odd split and zero otherwise)
    const std::uint32_t next_lo = ((hi ^ mask) << (c.wide - c.narrow)) | (lo >> c.narrow);
    hi = lo & narrow_mask;
    lo = next_lo;
  }
  return (static_cast<std::uint64_t>(hi) << c.wide) | lo;
}

struct image_under {
  index_cipher cipher;
  __host__ __device__ std::uint64_t operator()(std::uint64_t i) const { return encipher(cipher, i); }
};
struct falls_below {
  std::uint64_t m;
  __host__ __device__ bool operator()(std::uint64_t key) const { return key < m; }
};
// the input at a key; a key that is out of range is never kept, and reads element 0 meanwhile
template <typename It, typename V>
struct fetches_at {
  It in;
  std::uint64_t m;
  __host__ __device__ V operator()(std::uint64_t key) const { return in[key < m ? key : 0]; }
};

template <typename Keys, typename Policy, typename It, typename Out, typename URBG>
inline void shuffle_copy_with(Policy& exec, It first, It last, Out result, URBG&& g) {
  typedef typename std::remove_const<typename thrust::iterator_value<It>::type>::type V;
  const std::uint64_t m = (std::uint64_t)(last - first);
  const index_cipher cipher = make_index_cipher(m, g);  // (draws its keys also for an empty range, as the reference does)
  if (m == 0) return;
  const std::uint64_t n = cipher_domain(cipher);
  Keys keys(n);
  const image_under image = {cipher};
  thrust::transform(exec, thrust::counting_iterator<std::uint64_t>(0), thrust::counting_iterator<std::uint64_t>(n),
                    keys.begin(), image);
  const fetches_at<It, V> fetch = {first, m};
  const falls_below kept = {m};
  thrust::copy_if(exec, thrust::make_transform_iterator(keys.begin(), fetch),
                  thrust::make_transform_iterator(keys.end(), fetch), keys.begin(), result, kept);
}
}  // namespace detail

namespace system {
namespace cpp {
template <typename D, typename It, typename Out, typename URBG>
void shuffle_copy(execution_policy<D>& exec, It first, It last, Out result, URBG&& g) {
  thrust::detail::shuffle_copy_with<thrust::host_vector<std::uint64_t> >(exec, first, last, result, g);
}
template <typename D, typename It, typename URBG>
void shuffle(execution_policy<D>& exec, It first, It last, URBG&& g) {
  typedef typename std::remove_const<typename thrust::iterator_value<It>::type>::type V;
  const thrust::host_vector<V> from(first, last);
  thrust::detail::shuffle_copy_with<thrust::host_vector<std::uint64_t> >(exec, from.begin(), from.end(), first, g);
}
}  // namespace cpp
namespace hip {
template <typename D, typename It, typename Out, typename URBG>
void shuffle_copy(execution_policy<D>& exec, It first, It last, Out result, URBG&& g) {
  thrust::detail::shuffle_copy_with<thrust::device_vector<std::uint64_t> >(exec, first, last, result, g);
}
template <typename D, typename It, typename URBG>
void shuffle(execution_policy<D>& exec, It first, It last, URBG&& g) {
  typedef typename std::remove_const<typename thrust::iterator_value<It>::type>::type V;
  thrust::device_vector<V> from(last - first);
  thrust::copy(exec, first, last, from.begin());
  thrust::detail::shuffle_copy_with<thrust::device_vector<std::uint64_t> >(exec, from.begin(), from.end(), first, g);
}
}  // namespace hip
}  // namespace system

// ------------------------------------------------------------------ entry points
template <typename D, typename It, typename Out, typename URBG>
void shuffle_copy(const detail::execution_policy_base<D>& exec, It first, It last, Out result, URBG&& g) {
  shuffle_copy(detail::derived_cast(detail::strip_const(exec)), first, last, result, g);
}
template <typename It, typename Out, typename URBG,
          typename = typename std::enable_if<!detail::is_execution_policy<It>::value>::type>
void shuffle_copy(It first, It last, Out result, URBG&& g) {
  thrust::shuffle_copy(detail::policy_for<It>(), first, last, result, g);
}
template <typename D, typename It, typename URBG>
void shuffle(const detail::execution_policy_base<D>& exec, It first, It last, URBG&& g) {
  shuffle(detail::derived_cast(detail::strip_const(exec)), first, last, g);
}
template <typename It, typename URBG, typename = typename std::enable_if<!detail::is_execution_policy<It>::value>::type>
void shuffle(It first, It last, URBG&& g) {
  thrust::shuffle(detail::policy_for<It>(), first, last, g);
}

}  // namespace thrust
