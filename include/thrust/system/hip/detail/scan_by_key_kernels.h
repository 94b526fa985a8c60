// Single-pass segmented scan (inclusive_scan_by_key / exclusive_scan_by_key) as a template on
// the key equality and the operator.  A segment is a run of consecutive keys that the equality
// chains together.  libthrust_amd.so instantiates it for == and plus / minimum / maximum behind
// thrust_amd_inclusive_scan_by_key / thrust_amd_exclusive_scan_by_key; a translation unit
// compiled with hipcc instantiates it for its own equality and operator.
//
// Same machinery as reduce_by_key: every element carries the pair (heads, value) and
// pairs combine with (h1, v1) (+) (h2, v2) = (h1 + h2, h2 ? v2 : v1 OP v2); the scan runs
// lane -> wave (DPP) -> workgroup (LDS) -> grid (decoupled look-back, dynamic ticket),
// and here every element's inclusive value is written out.  The exclusive form writes
// init at a head and init OP (running value of the segment before the element) elsewhere:
// what the reference's scan of the right-shifted input with init at every head gives
// (thrust/system/detail/generic/scan_by_key.inl:216-234), out[i] = init OP v[s] OP ... OP v[i-1],
// without reading any element twice -- so that form, too, may write onto its input.
//
// Inside a segment the values are folded in a tree order: floating-point results agree
// with the reference's strict left fold (the OMP back end's scan is sequential,
// thrust/system/omp/detail/scan.h:21-22) only to rounding; integers are exact.
//
// HBM traffic: n*(key + value) read, n*value written.  Replaces the scan-by-key agent
// of thrust/system/cuda/detail/scan_by_key.h:203-830.
#pragma once
#include "reduce_by_key_kernels.h"

namespace thrust {
namespace system {
namespace hip {
namespace segmented {

constexpr int SBK_BLOCK = 512;  // two workgroups of 512 per CU

template <typename K, typename V, typename Eq, typename Op>
struct SbkArgs {
  const K* keys;
  const V* values;
  V* out;
  uint64_t n;
  V init;              // exclusive form only
  uint32_t exclusive;  // 0: inclusive, 1: exclusive
  uint64_t* status;
  uint32_t* ticket;
  uint32_t aligned;    // keys, values and out allow whole-vector accesses
  Eq eq;
  Op op;
};

// (a template only so that every translation unit may hold a copy)
template <int = 0>
__global__ __launch_bounds__(256) void sbk_init_kernel(uint64_t* __restrict__ words, uint64_t count,
                                                       uint32_t* __restrict__ ticket) {
  const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) words[i] = 0;
  if (i == 0) *ticket = 0;
}

// K is the key as the equality sees it.  The library passes an unsigned integer type of the
// key's size for integer keys (equal iff their bits are) and float / double for those.
template <typename K, typename V, typename Eq, typename Op>
__global__ __launch_bounds__(SBK_BLOCK, 4) void sbk_kernel(SbkArgs<K, V, Eq, Op> a) {
  constexpr int VEC = Vec16<K>::N;
  constexpr int CHUNKS = RBK_ITEMS / VEC >= 1 ? RBK_ITEMS / VEC : 1;
  constexpr int WAVES = SBK_BLOCK / WAVE;
  constexpr uint32_t WAVE_SPAN = WAVE * CHUNKS * VEC;
  constexpr uint32_t TILE = WAVES * WAVE_SPAN;
  using WV = typename SegValue<V>::type;
  using Pair = SegPair<WV>;
  using VV = RbkValueVec<V, VEC>;
  constexpr bool HAS_ID = names_identity<Op, V>::value;
  using ScanOp = SegScanOp<V, Op, HAS_ID>;
  const SegOp<V, Op> sop{a.op};
  const ScanOp scan_op{sop};
  // what stands in for elements past the end; with an identity also "nothing before this"
  V vid;
  if constexpr (HAS_ID) vid = Op::template identity<V>();
  else vid = V{};
  const Pair pid{HAS_ID ? 0u : RBK_EMPTY, (WV)vid};

  __shared__ uint32_t s_tile;
  __shared__ __attribute__((aligned(16))) unsigned char s_raw[(WAVES + 1) * sizeof(Pair)];  // values may be structs of the caller
  Pair* s_wave_agg = reinterpret_cast<Pair*>(s_raw);
  Pair& s_prefix = s_wave_agg[WAVES];

  if (threadIdx.x == 0) s_tile = atomicAdd(a.ticket, 1u);
  __syncthreads();
  const uint32_t tile = s_tile;
  const uint64_t tile_base = (uint64_t)tile * TILE;
  const uint32_t valid = (uint32_t)((a.n - tile_base < TILE) ? (a.n - tile_base) : TILE);
  const int wave = threadIdx.x / WAVE;
  const int lane = threadIdx.x % WAVE;
  const uint32_t lane_off = wave * WAVE_SPAN + lane * VEC;
  const bool full = valid == TILE;

  // ---- load
  Vec16<K> k[CHUNKS];
  VV v[CHUNKS];
  if (full && a.aligned) {
#pragma unroll
    for (int j = 0; j < CHUNKS; ++j) {
      const uint64_t off = tile_base + lane_off + j * (WAVE * VEC);
      k[j] = *reinterpret_cast<const Vec16<K>*>(a.keys + off);
      v[j] = *reinterpret_cast<const VV*>(a.values + off);
    }
  } else if (full) {
    // pointers that do not allow whole vectors: element loads, still without predicates
    // (a predicated load makes the compiler wait for it before issuing the next one)
#pragma unroll
    for (int j = 0; j < CHUNKS; ++j) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        const uint64_t off = tile_base + lane_off + j * (WAVE * VEC) + i;
        k[j].v[i] = a.keys[off];
        v[j].v[i] = a.values[off];
      }
    }
  } else {
#pragma unroll
    for (int j = 0; j < CHUNKS; ++j) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        const uint32_t e = lane_off + j * (WAVE * VEC) + i;
        k[j].v[i] = (e < valid) ? a.keys[tile_base + e] : K{};
        v[j].v[i] = (e < valid) ? a.values[tile_base + e] : vid;
      }
    }
  }

  // ---- head flags per chunk (bit i = element i); the exclusive form replaces the values
  // by their right-shifted neighbours with init at the heads; lane-local pairs
  uint32_t head[CHUNKS];
  Pair lane_excl[CHUNKS];
  Pair carry = pid;
#pragma unroll
  for (int j = 0; j < CHUNKS; ++j) {
    const uint64_t first = tile_base + lane_off + j * (WAVE * VEC);
    K prev = dpp_move<0x138 /* wave_shr:1 */>(k[j].v[VEC - 1], k[j].v[VEC - 1]);
    bool first_of_all = false;
    if (lane == 0) {
      if (first == 0) first_of_all = true;
      else if (first < a.n) prev = a.keys[first - 1];
    }
    uint32_t h = 0;
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      const K p = (i == 0) ? prev : k[j].v[i > 0 ? i - 1 : 0];
      const bool hd = (first + i < a.n) && ((i == 0 && first_of_all) || !a.eq(p, k[j].v[i]));
      h |= (uint32_t)hd << i;
    }
    head[j] = h;
    Pair agg{h & 1u, (WV)v[j].v[0]};
#pragma unroll
    for (int i = 1; i < VEC; ++i) agg = sop(agg, Pair{(h >> i) & 1u, (WV)v[j].v[i]});
    const Pair incl = wave_inclusive_scan(agg, scan_op, pid);
    lane_excl[j] = scan_op(carry, dpp_move<0x138>(pid, incl));
    carry = scan_op(carry, readlane(incl, WAVE - 1));
  }
  if (lane == 0) s_wave_agg[wave] = carry;
  // every load of this wave has returned before the tile's aggregate can become visible,
  // so the inclusive form may run in place (out == values)
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
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
  if (wave == 0) {
    Pair excl = pid;
    if (tile == 0) {
      if (lane == 0) tile_publish<Pair>(my_slot, TS_INCLUSIVE, tile_agg);
    } else {
      if (lane == 0) tile_publish<Pair>(my_slot, TS_PARTIAL, tile_agg);
      excl = tile_lookback<Pair>(a.status, tile, scan_op, pid);
      if (lane == 0) tile_publish<Pair>(my_slot, TS_INCLUSIVE, scan_op(excl, tile_agg));
    }
    if (lane == 0) s_prefix = excl;
  }
  __syncthreads();
  const Pair before_wave = scan_op(s_prefix, wave_prefix);

  // ---- every element's running value
#pragma unroll
  for (int j = 0; j < CHUNKS; ++j) {
    // (nothing at all before this lane: its first element is the very first one, a head)
    Pair run = scan_op(before_wave, lane_excl[j]);
    VV o;
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      const bool hd = (head[j] >> i) & 1u;
      // exclusive form: init at a head, else init combined with the running value of the
      // elements before this one in its segment (the element itself is folded in afterwards)
      if (a.exclusive) o.v[i] = hd ? a.init : (V)a.op(a.init, (V)run.value);
      run = sop(run, Pair{(uint32_t)hd, (WV)v[j].v[i]});
      if (!a.exclusive) o.v[i] = (V)run.value;
    }
    const uint32_t e0 = lane_off + j * (WAVE * VEC);
    if (full && a.aligned) {
      *reinterpret_cast<VV*>(a.out + tile_base + e0) = o;
    } else {
#pragma unroll
      for (int i = 0; i < VEC; ++i)
        if (e0 + i < valid) a.out[tile_base + e0 + i] = o.v[i];
    }
  }
}

// Temporary storage of one call: the tile ticket and the tile descriptors.
template <typename K, typename V>
struct SbkTemp {
  static constexpr int VEC = Vec16<K>::N;
  static constexpr int CHUNKS = RBK_ITEMS / VEC >= 1 ? RBK_ITEMS / VEC : 1;
  static constexpr uint64_t TILE = (uint64_t)SBK_BLOCK * CHUNKS * VEC;
  static constexpr int W = TileWords<SegPair<typename SegValue<V>::type> >::W;
  uint64_t tiles;
  size_t off_ticket, off_status, total;
  explicit SbkTemp(uint64_t n) : tiles((n + TILE - 1) / TILE) {
    TempLayout lay;
    off_ticket = lay.add(sizeof(uint32_t));
    off_status = lay.add((size_t)tiles * W * sizeof(uint64_t));
    total = lay.total;
  }
};

// Launches the init kernel and the scan into `temp` (SbkTemp<K, V>(n).total bytes); 0 < n < 2^32 - 1.
// Both forms may run in place (out == values): a tile stores only after all its loads have returned, and
// nothing outside the tile's own elements and the tile descriptors is read.
template <typename K, typename V, typename Eq, typename Op>
inline int sbk_launch(char* temp, const K* keys, const V* values, V* out, uint64_t n, bool exclusive, V init, Eq eq,
                      Op op, hipStream_t stream) {
  const SbkTemp<K, V> lay(n);
  if (lay.tiles > 0xffffffffull || n >= 0xffffffffull) return (int)hipErrorInvalidValue;
  constexpr size_t VALIGN = alignof(RbkValueVec<V, SbkTemp<K, V>::VEC>);
  SbkArgs<K, V, Eq, Op> a{keys,
                          values,
                          out,
                          n,
                          init,
                          exclusive ? 1u : 0u,
                          reinterpret_cast<uint64_t*>(temp + lay.off_status),
                          reinterpret_cast<uint32_t*>(temp + lay.off_ticket),
                          (is_aligned16(keys) && (reinterpret_cast<uintptr_t>(values) % VALIGN) == 0 &&
                           (reinterpret_cast<uintptr_t>(out) % VALIGN) == 0)
                              ? 1u
                              : 0u,
                          eq,
                          op};
  const uint64_t words = lay.tiles * SbkTemp<K, V>::W;
  THRUST_AMD_KERNEL_LAUNCH("sbk_init", stream, sbk_init_kernel<0>, dim3((uint32_t)((words + 255) / 256)), dim3(256),
                           a.status, words, a.ticket);
  hipError_t e = hipPeekAtLastError();
  if (e != hipSuccess) return (int)e;
  THRUST_AMD_KERNEL_LAUNCH("scan_by_key", stream, (sbk_kernel<K, V, Eq, Op>), dim3((uint32_t)lay.tiles), dim3(SBK_BLOCK),
                           a);
  return (int)hipPeekAtLastError();
}

}  // namespace segmented
}  // namespace hip
}  // namespace system
}  // namespace thrust
