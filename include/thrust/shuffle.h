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
// A keyed bijection of [0, 2^bits) (generic/shuffle.inl:34-140).
class feistel_bijection {
 public:
  template <typename URBG>
  __host__ __device__ feistel_bijection(std::uint64_t m, URBG&& g) {
    const std::uint64_t total_bits = cipher_bits(m);
    left_side_bits_ = total_bits / 2;
    left_side_mask_ = (1ull << left_side_bits_) - 1;
    right_side_bits_ = total_bits - left_side_bits_;
    right_side_mask_ = (1ull << right_side_bits_) - 1;
    for (int i = 0; i < ROUNDS; ++i) key_[i] = g();
  }
  __host__ __device__ std::uint64_t nearest_power_of_two() const { return 1ull << (left_side_bits_ + right_side_bits_); }
  __host__ __device__ std::uint64_t operator()(std::uint64_t val) const {
    std::uint32_t left = static_cast<std::uint32_t>(val >> right_side_bits_);
    std::uint32_t right = static_cast<std::uint32_t>(val & right_side_mask_);
    for (int i = 0; i < ROUNDS; ++i) {
      const std::uint32_t new_left = static_cast<std::uint32_t>(right & left_side_mask_);
      const std::uint32_t mixed = left ^ round_function(right, key_[i]);
      // an odd number of bits: the right side is one wider and keeps its top bit in place
      right = right_side_bits_ != left_side_bits_
                  ? static_cast<std::uint32_t>((static_cast<std::uint64_t>(mixed) << 1ull) | (right >> left_side_bits_))
                  : mixed;
      left = new_left;
    }
    return (static_cast<std::uint64_t>(left) << right_side_bits_) | right;
  }

 private:
  static const int ROUNDS = 16;
  __host__ __device__ static std::uint64_t cipher_bits(std::uint64_t m) {
    if (m == 0) return 0;
    std::uint64_t i = 0;
    for (--m; m != 0; m >>= 1) ++i;
    return i;
  }
  __host__ __device__ static std::uint64_t hash_combine(std::uint64_t lhs, std::uint64_t rhs) {
    lhs ^= rhs + 0x9e3779b9 + (lhs << 6) + (lhs >> 2);
    return lhs;
  }
  __host__ __device__ std::uint32_t round_function(std::uint64_t value, std::uint64_t key) const {
    const std::uint64_t hash0 = thrust::random::taus88(static_cast<std::uint32_t>(value))();
    const std::uint64_t hash1 = thrust::random::ranlux48(value)();
    return static_cast<std::uint32_t>(hash_combine(hash_combine(hash0, key), hash1) & left_side_mask_);
  }

  std::uint64_t right_side_bits_, left_side_bits_, right_side_mask_, left_side_mask_;
  std::uint64_t key_[ROUNDS];
};

struct image_under {
  feistel_bijection bijection;
  __host__ __device__ std::uint64_t operator()(std::uint64_t i) const { return bijection(i); }
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
  const feistel_bijection bijection(m, g);  // (draws its keys also for an empty range, as the reference does)
  if (m == 0) return;
  const std::uint64_t n = bijection.nearest_power_of_two();
  Keys keys(n);
  const image_under image = {bijection};
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
