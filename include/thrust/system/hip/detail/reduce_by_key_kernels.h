// Single-pass segmented reduction (reduce_by_key) as a template on the key equality and the
// operator.  libthrust_amd.so instantiates it for == and plus / minimum / maximum behind
// thrust_amd_reduce_by_key; a translation unit compiled with hipcc instantiates it for its own
// equality and operator, which then run inside the same kernel, as the reference passes them
// into its agent (thrust/system/cuda/detail/reduce_by_key.h:197-836).
//
// Every element carries the pair (heads, value): `heads` counts run beginnings, `value`
// is the fold of the values since the last run beginning.  Pairs combine with
//   (h1, v1) (+) (h2, v2) = (h1 + h2, h2 ? v2 : v1 OP v2)
// which is associative, so the same lane -> wave (DPP) -> workgroup (LDS) -> grid
// (decoupled look-back, dynamic tile ticket) scan as everywhere else applies.  With the
// inclusive pair (H, S) at element i: the run's first key goes to keys_out[H-1] at a run
// beginning, and the run total S goes to values_out[H-1] at a run end.
//
// An operator that names its identity (`Op::template identity<V>()`, as the library's do) uses
// it for "nothing before this".  Any other operator gets that case marked in the pair instead
// (heads == EMPTY), and the combination passes the other operand through.
//
// Inside a run the values are folded in a tree order, so floating-point sums agree
// with a strict left fold (the reference's OMP back end scans sequentially,
// thrust/system/omp/detail/scan.h:21-22) only to rounding.
//
// HBM traffic: n*(key + value) read, runs*(key + value) written, 8*W bytes of tile
// descriptor per tile.
#pragma once
#include "device_primitives.h"

namespace thrust {
namespace system {
namespace hip {
namespace segmented {
using namespace ::thrust::system::hip::prim;

// 16 elements per lane; the pair scan needs ~105 VGPRs, so a CU holds 16 waves.  For
// reduce_by_key one workgroup of 1024 threads measured best (large tiles keep the number of
// tiles in flight, and the look-back, small: 0.69 against 0.72 ms with 512 threads at 2^28
// pairs); scan_by_key, which also writes every element, prefers two workgroups of 512 that
// overlap each other's load, scan and store phases (0.71 against 0.79 ms).  reduce_by_key
// gives each lane 16 consecutive elements (one pair scan per wave); scan_by_key keeps the
// wave-striped vectors: with consecutive elements its 16-byte stores land 64 bytes apart
// and the kernel measured 0.81 ms.
constexpr int RBK_BLOCK = 1024;
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
  mutable Op op;  // a caller's operator need not be const-callable
  // value folds are done in the storage type V and widened only for transport
  using WV = typename SegValue<V>::type;
  THRUST_AMD_DEVICE SegPair<WV> operator()(const SegPair<WV>& a, const SegPair<WV>& b) const {
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

// Does the operator name its identity?
template <typename Op, typename V, typename = void>
struct names_identity : std::false_type {};
template <typename Op, typename V>
struct names_identity<Op, V, decltype((void)Op::template identity<V>())> : std::true_type {};

constexpr uint32_t RBK_EMPTY = 0xffffffffu;  // heads of "nothing before this" when the operator has no identity

// The pair operator as the scans use it: with an identity it is SegOp itself; without one an
// operand marked empty lets the other through.
template <typename V, typename Op, bool HAS_ID>
struct SegScanOp {
  SegOp<V, Op> sop;
  using Pair = SegPair<typename SegValue<V>::type>;
  THRUST_AMD_DEVICE Pair operator()(const Pair& a, const Pair& b) const {
    if constexpr (HAS_ID) {
      return sop(a, b);
    } else {
      const Pair both = sop(a, b);
      Pair r = (b.heads == RBK_EMPTY) ? a : both;
      if (a.heads == RBK_EMPTY) r = b;
      return r;
    }
  }
  // heads of a pair that may be the empty one
  static THRUST_AMD_DEVICE uint32_t heads(const Pair& p) { return (!HAS_ID && p.heads == RBK_EMPTY) ? 0u : p.heads; }
};

template <typename K, typename V, typename Eq, typename Op>
struct RbkArgs {
  const K* keys;
  const V* values;
  K* keys_out;
  V* values_out;
  uint64_t* d_num_runs;
  uint64_t n;
  uint64_t* status;
  uint32_t* ticket;
  uint32_t aligned;
  Eq eq;
  Op op;
};
// Arguments with every pointer null (the equality and the operator need not be default-constructible).
template <typename K, typename V, typename Eq, typename Op>
inline RbkArgs<K, V, Eq, Op> make_rbk_args(const Eq& eq, const Op& op) {
  return RbkArgs<K, V, Eq, Op>{nullptr, nullptr, nullptr, nullptr, nullptr, 0, nullptr, nullptr, 0u, eq, op};
}

// (a template only so that every translation unit may hold a copy)
template <int = 0>
__global__ __launch_bounds__(256) void rbk_init_kernel(uint64_t* __restrict__ words, uint64_t count,
                                                       uint32_t* __restrict__ ticket,
                                                       uint64_t* __restrict__ d_num) {
  const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) words[i] = 0;
  if (i == 0) {
    *ticket = 0;
    *d_num = 0;
  }
}

// Outputs of a tile with up to RBK_STAGED runs are gathered in LDS and leave in coalesced
// stores.  A tile with more runs writes them directly: its run beginnings are dense, so
// neighbouring lanes write neighbouring addresses anyway.
constexpr uint32_t RBK_STAGED = 4096;

// Shared memory of one workgroup, as raw bytes: keys and values may be structs of the caller.
template <typename K, typename V, typename Pair, int WAVES>
struct RbkShared {
  uint32_t tile;
  uint32_t first_is_head, last_is_tail;
  __attribute__((aligned(16))) unsigned char wave_agg[WAVES * sizeof(Pair)];
  __attribute__((aligned(16))) unsigned char prefix[sizeof(Pair)];
  __attribute__((aligned(16))) unsigned char keys_out[RBK_STAGED * sizeof(K)];
  __attribute__((aligned(16))) unsigned char values_out[(RBK_STAGED + 1) * sizeof(V)];
};

// K is the key as the equality sees it.  The library passes an unsigned integer type of the
// key's size for integer keys (equal iff their bits are) and float / double for those.
//
// Layout: a lane owns ITEMS = 16 or 28 consecutive elements (four or seven 16-byte key vectors
// for 4-byte keys), so the flags and the lane's fold are a serial pass over registers and the whole
// tile needs ONE wave scan of pairs per wave.  (Lanes of a wave then read 16-byte pieces
// 64 bytes apart; the loads of a lane cover its cache lines completely.)
template <typename K, typename V, typename Eq, typename Op>
__global__ __launch_bounds__((RbkItems<K, V>::block), 4) void rbk_kernel(RbkArgs<K, V, Eq, Op> a) {
  constexpr int BLOCK = RbkItems<K, V>::block;
  constexpr int VEC = Vec16<K>::N;
  constexpr int CHUNKS = RbkItems<K, V>::value / VEC >= 1 ? RbkItems<K, V>::value / VEC : 1;
  constexpr int ITEMS = CHUNKS * VEC;
  constexpr int WAVES = BLOCK / WAVE;
  constexpr uint32_t TILE = BLOCK * ITEMS;
  constexpr bool HAS_ID = names_identity<Op, V>::value;
  using WV = typename SegValue<V>::type;
  using Pair = SegPair<WV>;
  using VV = RbkValueVec<V, VEC>;
  using ScanOp = SegScanOp<V, Op, HAS_ID>;
  const SegOp<V, Op> sop{a.op};
  const ScanOp scan_op{sop};
  // what stands in for elements past the end; with an identity also "nothing before this"
  V vid;
  if constexpr (HAS_ID) vid = Op::template identity<V>();
  else vid = V{};
  const Pair pid{HAS_ID ? 0u : RBK_EMPTY, (WV)vid};

  __shared__ RbkShared<K, V, Pair, WAVES> sh;
  Pair* s_wave_agg = reinterpret_cast<Pair*>(sh.wave_agg);
  Pair* s_prefix = reinterpret_cast<Pair*>(sh.prefix);
  K* s_keys_out = reinterpret_cast<K*>(sh.keys_out);
  V* s_values_out = reinterpret_cast<V*>(sh.values_out);

  if (threadIdx.x == 0) sh.tile = atomicAdd(a.ticket, 1u);
  __syncthreads();
  const uint32_t tile = sh.tile;
  const uint64_t tile_base = (uint64_t)tile * TILE;
  const uint32_t valid = (uint32_t)((a.n - tile_base < TILE) ? (a.n - tile_base) : TILE);
  const int wave = threadIdx.x / WAVE;
  const int lane = threadIdx.x % WAVE;
  const uint32_t lane_off = threadIdx.x * ITEMS;
  const uint64_t first = tile_base + lane_off;  // global index of the lane's first element
  const bool full = valid == TILE;

  // ---- load
  K k[ITEMS];
  V v[ITEMS];
  if (full && a.aligned) {
    Vec16<K> kv[CHUNKS];
    VV vv[CHUNKS];
#pragma unroll
    for (int j = 0; j < CHUNKS; ++j) {
      kv[j] = *reinterpret_cast<const Vec16<K>*>(a.keys + first + j * VEC);
      vv[j] = *reinterpret_cast<const VV*>(a.values + first + j * VEC);
    }
#pragma unroll
    for (int j = 0; j < CHUNKS; ++j) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        k[j * VEC + i] = kv[j].v[i];
        v[j * VEC + i] = vv[j].v[i];
      }
    }
  } else if (full) {
    // pointers that do not allow whole vectors: element loads, still without predicates
    // (a predicated load makes the compiler wait for it before issuing the next one)
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
      k[i] = a.keys[first + i];
      v[i] = a.values[first + i];
    }
  } else {
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
      const uint32_t e = lane_off + i;
      k[i] = (e < valid) ? a.keys[tile_base + e] : K{};
      v[i] = (e < valid) ? a.values[tile_base + e] : vid;
    }
  }

  // ---- head / tail flags (bit i = element i) and the fold of the lane's elements
  K prev = dpp_move<0x138 /* wave_shr:1 */>(k[ITEMS - 1], k[ITEMS - 1]);
  K next = dpp_move<0x130 /* wave_shl:1 */>(k[0], k[0]);
  if (lane == 0 && first > 0 && first < a.n) prev = a.keys[first - 1];
  if (lane == WAVE - 1 && first + ITEMS < a.n) next = a.keys[first + ITEMS];
  // differs[i]: element i differs from its predecessor; bit ITEMS: the lane's successor differs
  uint32_t differs = 0;
#pragma unroll
  for (int i = 0; i < ITEMS; ++i) differs |= (uint32_t)(!a.eq((i == 0) ? prev : k[i > 0 ? i - 1 : 0], k[i])) << i;
  differs |= (uint32_t)(!a.eq(k[ITEMS - 1], next)) << ITEMS;
  if (tile == 0 && threadIdx.x == 0) differs |= 1u;  // the very first element starts a run
  const uint32_t live = (lane_off >= valid) ? 0u
                        : ((valid - lane_off >= (uint32_t)ITEMS) ? ((1u << ITEMS) - 1u) : ((1u << (valid - lane_off)) - 1u));
  // the very last element ends a run (it is in the last tile, at local index valid - 1)
  const bool last_tile = tile_base + valid == a.n;
  const uint32_t last_bit = (last_tile && valid - 1 >= lane_off && valid - 1 - lane_off < (uint32_t)ITEMS)
                                ? (1u << (valid - 1 - lane_off)) : 0u;
  const uint32_t head = differs & live;
  const uint32_t tail = ((differs >> 1) | last_bit) & live;
  Pair agg{head & 1u, (WV)v[0]};
#pragma unroll
  for (int i = 1; i < ITEMS; ++i) agg = sop(agg, Pair{(head >> i) & 1u, (WV)v[i]});
  const Pair incl = wave_inclusive_scan(agg, scan_op, pid);
  const Pair lane_excl = dpp_move<0x138>(pid, incl);
  if (lane == WAVE - 1) s_wave_agg[wave] = incl;
  __syncthreads();
  Pair wave_prefix = pid, tile_agg = pid;
#pragma unroll
  for (int w = 0; w < WAVES; ++w) {
    if (w == wave) wave_prefix = tile_agg;
    tile_agg = scan_op(tile_agg, s_wave_agg[w]);
  }

  // ---- pair of everything before this tile
  constexpr int W = TileWords<Pair>::W;
  uint64_t* my_slot = a.status + (size_t)tile * W;
  if (wave == 0 && lane == 0) tile_publish<Pair>(my_slot, tile == 0 ? TS_INCLUSIVE : TS_PARTIAL, tile_agg);

  // Outputs of a tile with up to RBK_STAGED runs are gathered in LDS at their place inside the
  // tile -- which needs nothing from earlier tiles -- while the prefix is on its way; only the
  // total of a run that began in an earlier tile and ends here is completed afterwards
  // (0.617 -> 0.544 ms at 2^28 pairs with a mean run of 8: what a tile does after its prefix has
  // arrived is what every later tile waits for).
  const uint32_t tile_runs = tile_agg.heads;  // runs begun in this tile
  const bool staged = tile_runs <= RBK_STAGED;
  if (staged) {
    // Run r of the tile (0-based) keeps its key in slot r and its total in slot r + 1: slot 0 of
    // the totals belongs to the run that began before the tile.
    if (threadIdx.x == 0) sh.first_is_head = head & 1u;
    if (valid - 1 >= lane_off && valid - 1 - lane_off < (uint32_t)ITEMS) sh.last_is_tail = (tail >> (valid - 1 - lane_off)) & 1u;
    Pair run = scan_op(wave_prefix, lane_excl);  // of the tile's elements before this lane
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
      run = scan_op(run, Pair{(head >> i) & 1u, (WV)v[i]});
      if ((head >> i) & 1u) s_keys_out[run.heads - 1] = k[i];
      if ((tail >> i) & 1u) s_values_out[run.heads] = (V)run.value;
    }
  }

  if (wave == 0) {
    Pair excl = pid;
    if (tile != 0) {
      excl = tile_lookback<Pair, 16>(a.status, tile, scan_op, pid);
      if (lane == 0) tile_publish<Pair>(my_slot, TS_INCLUSIVE, scan_op(excl, tile_agg));
    }
    if (lane == 0) {
      *s_prefix = excl;
      if (tile_base + valid == a.n) *a.d_num_runs = (uint64_t)ScanOp::heads(excl) + tile_agg.heads;
    }
  }
  __syncthreads();

  // ---- emit first keys at run beginnings, run totals at run ends
  const uint32_t runs_before = ScanOp::heads(*s_prefix);  // runs begun before this tile
  if (!staged) {
    // many runs: written where they belong directly
    Pair run = scan_op(scan_op(*s_prefix, wave_prefix), lane_excl);
    // nothing at all before this lane: its first element is the very first one and starts a run
    if (!HAS_ID && run.heads == RBK_EMPTY) run.heads = 0;
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
      run = sop(run, Pair{(head >> i) & 1u, (WV)v[i]});
      if ((head >> i) & 1u) a.keys_out[run.heads - 1] = k[i];
      if ((tail >> i) & 1u) a.values_out[run.heads - 1] = (V)run.value;
    }
    return;
  }
  for (uint32_t j = threadIdx.x; j < tile_runs; j += BLOCK) a.keys_out[(uint64_t)runs_before + j] = s_keys_out[j];
  // totals present: every run touched by the tile except a last one that goes on
  const uint32_t lo = sh.first_is_head ? 1u : 0u;
  const uint32_t hi = sh.last_is_tail ? tile_runs + 1u : tile_runs;  // exclusive
  for (uint32_t j = lo + threadIdx.x; j < hi; j += BLOCK) {
    V total = s_values_out[j];
    // the run from before the tile: what earlier tiles hold of it comes first
    if (j == 0) total = (V)sop.op((V)s_prefix->value, total);
    a.values_out[(uint64_t)runs_before + j - 1] = total;
  }
}

// Temporary storage of one call: the tile ticket and the tile descriptors.
template <typename K, typename V>
struct RbkTemp {
  static constexpr int VEC = Vec16<K>::N;
  static constexpr int CHUNKS = RbkItems<K, V>::value / VEC >= 1 ? RbkItems<K, V>::value / VEC : 1;
  static constexpr int BLOCK = RbkItems<K, V>::block;
  static constexpr uint64_t TILE = (uint64_t)BLOCK * CHUNKS * VEC;
  static constexpr int W = TileWords<SegPair<typename SegValue<V>::type> >::W;
  uint64_t tiles;
  size_t off_ticket, off_status, total;
  explicit RbkTemp(uint64_t n) : tiles((n + TILE - 1) / TILE) {
    TempLayout lay;
    off_ticket = lay.add(sizeof(uint32_t));
    off_status = lay.add((size_t)tiles * W * sizeof(uint64_t));
    total = lay.total;
  }
};

// Launches the init kernel and the reduction into `temp` (RbkTemp<K, V>(n).total bytes).
// a.keys .. a.n, a.eq and a.op are the caller's; n < 2^32 - 1.
template <typename K, typename V, typename Eq, typename Op>
inline int rbk_launch(char* temp, RbkArgs<K, V, Eq, Op> a, hipStream_t stream) {
  const RbkTemp<K, V> lay(a.n);
  if (lay.tiles > 0xffffffffull || a.n >= 0xffffffffull) return (int)hipErrorInvalidValue;
  a.ticket = reinterpret_cast<uint32_t*>(temp + lay.off_ticket);
  a.status = reinterpret_cast<uint64_t*>(temp + lay.off_status);
  a.aligned = is_aligned16(a.keys) &&
              (reinterpret_cast<uintptr_t>(a.values) % alignof(RbkValueVec<V, RbkTemp<K, V>::VEC>)) == 0;
  const uint64_t words = lay.tiles * RbkTemp<K, V>::W;
  const uint64_t init_threads = words ? words : 1;
  THRUST_AMD_KERNEL_LAUNCH("rbk_init", stream, rbk_init_kernel<0>, dim3((uint32_t)((init_threads + 255) / 256)), dim3(256),
                           a.status, words, a.ticket, a.d_num_runs);
  hipError_t e = hipPeekAtLastError();
  if (e != hipSuccess) return (int)e;
  if (a.n == 0) return 0;
  THRUST_AMD_KERNEL_LAUNCH("reduce_by_key", stream, (rbk_kernel<K, V, Eq, Op>), dim3((uint32_t)lay.tiles),
                           dim3(RbkTemp<K, V>::BLOCK), a);
  return (int)hipPeekAtLastError();
}

}  // namespace segmented
}  // namespace hip
}  // namespace system
}  // namespace thrust
