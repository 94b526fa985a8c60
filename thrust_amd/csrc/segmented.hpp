// Pieces shared by the segmented single-pass kernels (reduce_by_key, scan_by_key): the
// (heads, value) pair, its associative operator, the value vector that travels with a
// 16-byte vector of keys, and the tile shape.
#pragma once
#include "common.hpp"

namespace ta {

// 16 elements per lane; the pair scan needs ~105 VGPRs, so a CU holds 16 waves.  For
// reduce_by_key one workgroup of 1024 threads measured best (large tiles keep the number of
// tiles in flight, and the look-back, small: 0.69 against 0.72 ms with 512 threads at 2^28
// pairs); scan_by_key, which also writes every element, prefers two workgroups of 512 that
// overlap each other's load, scan and store phases (0.71 against 0.79 ms).  reduce_by_key
// gives each lane 16 consecutive elements (one pair scan per wave); scan_by_key keeps the
// wave-striped vectors: with consecutive elements its 16-byte stores land 64 bytes apart
// and the kernel measured 0.81 ms.
constexpr int RBK_BLOCK = 1024;
constexpr int SBK_BLOCK = 512;
constexpr int RBK_ITEMS = 16;  // elements per lane

// reduce_by_key with keys and values of up to four bytes: 512 threads x 28 elements per lane,
// two workgroups per CU (127 registers) -- more bytes per CU wait for their prefix at a time
// than with one workgroup of 1024 x 20 (0.65 -> 0.61 ms and 0.61 -> 0.57 ms at 2^28 pairs,
// mean run 8 / 1000; 1024 x 24 spills and loses).  Wider elements stay at 1024 x 16.
template <typename K, typename V>
struct RbkItems {
  static constexpr bool NARROW = sizeof(K) <= 4 && sizeof(V) <= 4;
  static constexpr int value = NARROW ? 28 : RBK_ITEMS;
  static constexpr int block = NARROW ? 512 : RBK_BLOCK;
};

template <typename V>
struct alignas(sizeof(V) >= 8 ? 8 : 4) SegPair {
  uint32_t heads;
  V value;
};
// 1- and 2-byte values are widened so that the pair is a whole number of 32-bit words.
template <typename V> struct SegValue { using type = V; };
template <> struct SegValue<int8_t> { using type = int32_t; };
template <> struct SegValue<uint8_t> { using type = uint32_t; };
template <> struct SegValue<int16_t> { using type = int32_t; };
template <> struct SegValue<uint16_t> { using type = uint32_t; };

template <typename V, typename Op>
struct SegOp {
  Op op;
  // value folds are done in the storage type V and widened only for transport
  using WV = typename SegValue<V>::type;
  TA_DEVICE SegPair<WV> operator()(const SegPair<WV>& a, const SegPair<WV>& b) const {
    SegPair<WV> r;
    r.heads = a.heads + b.heads;
    r.value = b.heads ? b.value : (WV)op((V)a.value, (V)b.value);
    return r;
  }
};

template <typename V, int VEC>
struct alignas((VEC * sizeof(V)) >= 16 ? 16 : VEC * sizeof(V)) RbkValueVec {
  V v[VEC];
};

}  // namespace ta
