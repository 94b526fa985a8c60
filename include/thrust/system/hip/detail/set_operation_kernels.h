// set_difference, set_intersection, set_symmetric_difference and set_union of two sorted ranges
// (and their by_key forms) with multiset semantics, in one pass over the merge path, as
// templates on the comparator.  libthrust_amd.so instantiates them for operator< / operator>
// behind thrust_amd_set_operation / thrust_amd_set_operation_by_key; a translation unit compiled
// with hipcc instantiates them for its own comparator and key type.
//
// For a key x that occurs m times in A and n times in B, the merged order (A first on
// ties) holds the run A_0 .. A_{m-1} B_0 .. B_{n-1}, and the reference's sequential loops
// (thrust/system/detail/sequential/set_operations.h:42-215) keep, in that order,
//   difference            A_r with r >= n
//   intersection          A_r with r <  n
//   symmetric difference  A_r with r >= n and B_r with r >= m
//   union                 every A_r     and B_r with r >= m
// so an element is decided by its rank r inside its own part of the run and by the size
// of the other part.  Both follow from three positions per run on the merge path: where
// the run starts, where its B part starts and where it ends.
//
//   partition  one thread per tile boundary: the merge-path split, and the three
//              positions (by binary search over the whole ranges) of the run that
//              contains the first element of the tile -- the only run of a tile that can
//              start before it, and, read from the next boundary, the only one that can
//              end after it
//   tile       stages its two sub-ranges in LDS and merges them serially per lane as
//              the merge kernel does; head flags on the merged order and two workgroup scans
//              (last / next run start and B-part start) give the three positions of
//              every interior run; keep flags -> ranks -> decoupled look-back over the
//              tiles' counts (dynamic tickets) -> compaction through LDS -> coalesced
//              stores; values are gathered from the range their key came from
//
// Equivalent keys need not be identical (-0.0 and +0.0 under operator<), the copy that is kept is the one the rule above names.
// HBM traffic: (na + nb) keys read, the result written, values read only where kept.
// Replaces the balanced-path SetOpAgent of thrust/system/cuda/detail/set_operations.h:224-1330.
#pragma once
#include "device_primitives.h"

namespace thrust {
namespace system {
namespace hip {
namespace setops {
using namespace ::thrust::system::hip::prim;

// Tile = BLOCK threads x 16 merged elements each: 8192 elements for keys and values of up
// to 4 bytes, 4096 for 8-byte items.  Tiles take dynamic tickets (a same-address atomic
// retires about every 12 ns) and chain their counts, which favours large tiles; two
// workgroups per CU hide each other's barriers, which caps them (16384-element tiles of
// 1024 threads measured slower than these).
constexpr int SET_ITEMS = 16;
template <typename T, typename V, bool HAS_VALUES>
struct SetShape {
  static constexpr size_t ITEM = (HAS_VALUES && sizeof(V) > sizeof(T)) ? sizeof(V) : sizeof(T);
  static constexpr int BLOCK = ITEM > 4 ? 256 : 512;
  static constexpr int TILE = BLOCK * SET_ITEMS;
  // waves per SIMD the register allocation aims at: the merge of 8-byte items does not fit
  // the 128 registers that four would leave
  static constexpr int WAVES_PER_SIMD = ITEM > 4 ? 3 : 4;
};

// Number of elements taken from A among the first `diag` elements of the merged order.
template <typename T, typename PA, typename PB, typename Comp>
THRUST_AMD_DEVICE uint64_t set_merge_path(PA a, uint64_t na, PB b, uint64_t nb, uint64_t diag, Comp& comp) {
  uint64_t lo = diag > nb ? diag - nb : 0;
  uint64_t hi = diag < na ? diag : na;
  while (lo < hi) {
    const uint64_t mid = (lo + hi) >> 1;
    if (!comp(b[diag - 1 - mid], a[mid])) lo = mid + 1;
    else hi = mid;
  }
  return lo;
}

// Per tile boundary t (t = 0 .. tiles), found by one thread: split[t] = elements of A before
// merged position t * tile_size; for boundaries inside the merged order, key[t] = the
// element at that position and run[3t .. 3t+2] = merged positions where its run starts,
// where the run's B part starts, and where the run ends.
template <typename T, typename Comp>
__global__ __launch_bounds__(256) void set_partition_kernel(const T* __restrict__ a, uint64_t na,
                                                            const T* __restrict__ b, uint64_t nb,
                                                            uint64_t tiles, uint32_t tile_size,
                                                            Comp comp,
                                                            uint64_t* __restrict__ split,
                                                            uint64_t* __restrict__ run,
                                                            T* __restrict__ key) {
  const uint64_t t = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t > tiles) return;
  const uint64_t total = na + nb;
  uint64_t diag = t * tile_size;
  if (diag > total) diag = total;
  const uint64_t as = aligned_partition_point(diag > nb ? diag - nb : 0, diag < na ? diag : na, [&](uint64_t mid) {
    return !comp(b[diag - 1 - mid], a[mid]);
  });
  split[t] = as;
  if (diag >= total) return;
  const uint64_t bs = diag - as;
  T x;
  if (as < na && (bs >= nb || !comp(b[bs], a[as]))) x = a[as];
  else x = b[bs];
  // first index whose element is not before x / is after x, in each range
  const uint64_t lb_a = aligned_partition_point(0, na, [&](uint64_t i) { return comp(a[i], x); });
  const uint64_t ub_a = aligned_partition_point(lb_a, na, [&](uint64_t i) { return !comp(x, a[i]); });
  const uint64_t lb_b = aligned_partition_point(0, nb, [&](uint64_t i) { return comp(b[i], x); });
  const uint64_t ub_b = aligned_partition_point(lb_b, nb, [&](uint64_t i) { return !comp(x, b[i]); });
  key[t] = x;
  run[3 * t + 0] = lb_a + lb_b;
  run[3 * t + 1] = ub_a + lb_b;
  run[3 * t + 2] = ub_a + ub_b;
}

// (a template only so that every translation unit may hold a copy)
template <int = 0>
__global__ __launch_bounds__(256) void set_init_kernel(uint64_t* __restrict__ words, uint64_t count,
                                                       uint32_t* __restrict__ ticket,
                                                       uint64_t* __restrict__ d_num) {
  const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) words[i] = 0;
  if (i == 0) {
    *ticket = 0;
    *d_num = 0;
  }
}

// Two positions scanned together: the run start in the high half, the B-part start in the low.
struct OpMaxPair {
  THRUST_AMD_DEVICE uint64_t operator()(uint64_t x, uint64_t y) const {
    const uint32_t xh = (uint32_t)(x >> 32), yh = (uint32_t)(y >> 32);
    const uint32_t xl = (uint32_t)x, yl = (uint32_t)y;
    return ((uint64_t)(xh > yh ? xh : yh) << 32) | (xl > yl ? xl : yl);
  }
};

// Fold of the values of all threads before this one (`id` for thread 0) in a workgroup of
// WAVES waves.  `buf` holds WAVES values; the caller separates uses of it with a barrier.
template <int WAVES, typename V, typename Op>
THRUST_AMD_DEVICE V set_block_exclusive(V v, Op op, V id, V* buf, V* total) {
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const V incl = wave_inclusive_scan(v, op, id);
  if (lane == WAVE - 1) buf[wave] = incl;
  __syncthreads();
  V prefix = id, all = id;
#pragma unroll
  for (int w = 0; w < WAVES; ++w) {
    if (w == wave) prefix = all;
    all = op(all, buf[w]);
  }
  if (total) *total = all;
  const V before = dpp_move<0x138 /* wave_shr:1 */>(id, incl);
  return op(prefix, before);
}

template <typename T, typename V, bool HAS_VALUES, typename Comp>
struct SetArgs {
  const T* a;
  const T* b;
  const V* va;
  const V* vb;
  T* out;
  V* vout;
  uint64_t na, nb;
  const uint64_t* split;
  const uint64_t* run;
  const T* key;
  uint64_t* status;
  uint32_t* ticket;
  uint64_t* d_num;
  uint64_t tiles;
  int op;
  Comp comp;
};

template <typename T, typename V, bool HAS_VALUES, typename Comp>
__global__ __launch_bounds__((SetShape<T, V, HAS_VALUES>::BLOCK), (SetShape<T, V, HAS_VALUES>::WAVES_PER_SIMD)) void set_op_kernel(SetArgs<T, V, HAS_VALUES, Comp> g) {
  using Shape = SetShape<T, V, HAS_VALUES>;
  constexpr int SET_BLOCK = Shape::BLOCK;
  constexpr int SET_TILE = Shape::TILE;
  constexpr int SET_WAVES = SET_BLOCK / WAVE;
  // one buffer for the staged keys, the compacted keys and (later) the staged values
  __shared__ __attribute__((aligned(16))) unsigned char s_raw[(size_t)(SET_TILE + 1) * Shape::ITEM];
  T* s_keys = reinterpret_cast<T*>(s_raw);
  V* s_vals = reinterpret_cast<V*>(s_raw);
  __shared__ uint16_t s_src[HAS_VALUES ? SET_TILE : 1];
  __shared__ __attribute__((aligned(16))) unsigned char s_edge_raw[SET_BLOCK * sizeof(T)];  // keys may be structs of the caller
  T* s_edge_key = reinterpret_cast<T*>(s_edge_raw);
  __shared__ uint8_t s_edge_b[SET_BLOCK];
  __shared__ uint64_t s_pair[SET_BLOCK];
  __shared__ uint64_t s_scan64[SET_WAVES];
  __shared__ uint32_t s_scan32[SET_WAVES];
  __shared__ uint32_t s_tile;
  __shared__ uint64_t s_base;

  Comp& comp = g.comp;
  if (threadIdx.x == 0) s_tile = atomicAdd(g.ticket, 1u);
  __syncthreads();
  const uint64_t tile = s_tile;
  const uint64_t total = g.na + g.nb;
  const uint64_t d0 = tile * SET_TILE;
  const uint64_t d1 = (d0 + SET_TILE < total) ? d0 + SET_TILE : total;
  const uint64_t a0 = g.split[tile], a1 = g.split[tile + 1];
  const uint64_t b0 = d0 - a0, b1 = d1 - a1;
  const uint32_t ca = (uint32_t)(a1 - a0), cb = (uint32_t)(b1 - b0);
  const uint32_t count = ca + cb;  // == d1 - d0, 1 .. SET_TILE

  // The run the tile starts in, and the run the next tile starts in (the only runs that can
  // reach outside the tile).  With rs / rm / re the merged positions where such a run
  // starts, where its B part starts and where it ends, its element at merged position P
  // has rank P - rs >= (re - rm) [A] or P - rm >= (rm - rs) [B] exactly when its tile-local
  // position is at or past a threshold that is the same for the whole tile.
  const T f0_key = g.key[tile];
  const bool f1_valid = d1 < total;
  const T f1_key = f1_valid ? g.key[tile + 1] : f0_key;
  auto local_threshold = [&](uint64_t global_pos) -> uint32_t {
    if (global_pos <= d0) return 0u;
    const uint64_t rel = global_pos - d0;
    return rel > (uint64_t)SET_TILE ? (uint32_t)SET_TILE + 1u : (uint32_t)rel;
  };
  uint32_t thr_a0, thr_b0, thr_a1 = 0, thr_b1 = 0;
  {
    const uint64_t rs = g.run[3 * tile], rm = g.run[3 * tile + 1], re = g.run[3 * tile + 2];
    thr_a0 = local_threshold(rs + (re - rm));
    thr_b0 = local_threshold(rm + (rm - rs));
  }
  if (f1_valid) {
    const uint64_t rs = g.run[3 * (tile + 1)], rm = g.run[3 * (tile + 1) + 1], re = g.run[3 * (tile + 1) + 2];
    thr_a1 = local_threshold(rs + (re - rm));
    thr_b1 = local_threshold(rm + (rm - rs));
  }

  // ---- stage the keys: A's part first, then B's
  {
    T in[SET_ITEMS];
#pragma unroll
    for (int q = 0; q < SET_ITEMS; ++q) {
      const uint32_t e = q * SET_BLOCK + threadIdx.x;
      in[q] = (e < ca) ? g.a[a0 + e] : (e < count) ? g.b[b0 + (e - ca)] : T{};
    }
#pragma unroll
    for (int q = 0; q < SET_ITEMS; ++q) s_keys[q * SET_BLOCK + threadIdx.x] = in[q];
    if (threadIdx.x == 0) s_keys[SET_TILE] = T{};
  }
  __syncthreads();

  // ---- this lane's start on the path, then a serial merge of ITEMS elements
  const uint32_t run0 = threadIdx.x * SET_ITEMS;
  const uint32_t diag = run0 < count ? run0 : count;
  uint32_t i = (uint32_t)set_merge_path<T>(s_keys, (uint64_t)ca, s_keys + ca, (uint64_t)cb, (uint64_t)diag, comp);
  uint32_t j = ca + (diag - i);
  T k[SET_ITEMS];
  uint32_t slot[SET_ITEMS];
  uint32_t is_b = 0;  // bit o: merged element o of this lane comes from B
  {
    T ka = s_keys[i];
    T kb = s_keys[j];
#pragma unroll
    for (int o = 0; o < SET_ITEMS; ++o) {
      const bool take_b = (j < count) && (i >= ca || comp(kb, ka));
      k[o] = take_b ? kb : ka;
      slot[o] = take_b ? j : i;
      is_b |= (uint32_t)take_b << o;
      const uint32_t next = take_b ? ++j : ++i;
      const T nk = s_keys[next];  // next <= count <= SET_TILE
      if (take_b) kb = nk;
      else ka = nk;
    }
  }
  // valid elements of this lane: merged positions run0 + o < count
  const uint32_t live = (run0 >= count) ? 0u : ((count - run0 >= (uint32_t)SET_ITEMS) ? 0xffffu : ((1u << (count - run0)) - 1u));

  // does the tile's last run go on in the next tile?  (the last merged key is the later of
  // the two parts' last keys; only its equivalence class matters)
  bool tail_continues = false;
  if (f1_valid) {
    const T last_a = s_keys[ca ? ca - 1 : 0], last_b = s_keys[count - 1];
    const T last = (cb == 0) ? last_a : (ca == 0) ? last_b : (comp(last_b, last_a) ? last_a : last_b);
    tail_continues = !comp(last, f1_key);
  }

  // ---- head flags on the merged order: bit o set when valid element o starts a run (local
  // position 0 counts as a start); e2: first B of a run
  s_edge_key[threadIdx.x] = k[SET_ITEMS - 1];
  s_edge_b[threadIdx.x] = (uint8_t)((is_b >> (SET_ITEMS - 1)) & 1u);
  __syncthreads();
  uint32_t head = 0;
  {
    T prev = (threadIdx.x > 0) ? s_edge_key[threadIdx.x - 1] : k[0];
#pragma unroll
    for (int o = 0; o < SET_ITEMS; ++o) {
      head |= (uint32_t)comp(prev, k[o]) << o;
      prev = k[o];
    }
    if (threadIdx.x == 0) head |= 1u;
    head &= live;
  }
  // first B of a run: a B whose predecessor is an A, or that starts a run
  const uint32_t prev_b_bits = (is_b << 1) | ((threadIdx.x > 0) ? (uint32_t)s_edge_b[threadIdx.x - 1] : 0u);
  const uint32_t e2 = is_b & (head | ~prev_b_bits) & live;

  // ---- last run start / B-part start at or before each element (forward scan), next ones
  // after it (backward scan).  Positions are stored +1 so that 0 means "none" in the forward
  // scan; the backward scan runs over mirrored positions (SET_TILE - p) and mirrored lanes.
  uint64_t fwd_in, bwd_in, fwd_all, bwd_all;
  {
    const uint32_t head_after0 = (threadIdx.x == 0) ? (head & ~1u) : head;  // position 0 is never "next"
    const uint32_t last_h = head ? run0 + (31 - __builtin_clz(head)) + 1 : 0u;
    const uint32_t last_e2 = e2 ? run0 + (31 - __builtin_clz(e2)) + 1 : 0u;
    const uint32_t first_h = head_after0 ? SET_TILE - (run0 + __builtin_ctz(head_after0)) : 0u;
    const uint32_t first_e2 = e2 ? SET_TILE - (run0 + __builtin_ctz(e2)) : 0u;
    fwd_in = set_block_exclusive<SET_WAVES, uint64_t>(((uint64_t)last_h << 32) | last_e2, OpMaxPair{}, (uint64_t)0,
                                                      s_scan64, &fwd_all);
    // mirrored lanes: thread t contributes as thread BLOCK - 1 - t
    s_pair[SET_BLOCK - 1 - threadIdx.x] = ((uint64_t)first_h << 32) | first_e2;
    __syncthreads();
    const uint64_t mirrored = s_pair[threadIdx.x];
    __syncthreads();  // s_scan64 and s_pair are reused below
    const uint64_t r = set_block_exclusive<SET_WAVES, uint64_t>(mirrored, OpMaxPair{}, (uint64_t)0, s_scan64, &bwd_all);
    s_pair[SET_BLOCK - 1 - threadIdx.x] = r;
    __syncthreads();
    bwd_in = s_pair[threadIdx.x];
  }
  // the first run of the tile ends where the first later run starts; the last run starts at
  // the last run start (position 0 is one, so there always is one)
  const uint32_t first_end = (uint32_t)(bwd_all >> 32) ? SET_TILE - (uint32_t)(bwd_all >> 32) : count;
  const uint32_t last_start = (uint32_t)(fwd_all >> 32) - 1u;

  // ---- decide every element
  // backward pass: the number of B elements of the element's run that lie after it (for an
  // element of A that is the size of the run's B part, because all of them follow it);
  // two 16-bit counts per register
  uint32_t b_after[SET_ITEMS / 2];
  {
    // mirrored value v = SET_TILE - p, 0 = none  ->  position, `count` when there is none
    const uint32_t nh = (uint32_t)(bwd_in >> 32), ne = (uint32_t)bwd_in;
    uint32_t cur_h = nh ? SET_TILE - nh : count;  // next run start after this element
    uint32_t cur_e = ne ? SET_TILE - ne : count;  // next B-part start after this element
#pragma unroll
    for (int o = SET_ITEMS - 1; o >= 0; --o) {
      const uint32_t nb_run = (cur_e < cur_h) ? cur_h - cur_e : 0u;
      if (o & 1) b_after[o / 2] = nb_run << 16;
      else b_after[o / 2] |= nb_run;
      const uint32_t p = run0 + o;
      if ((head >> o) & 1u) cur_h = p;
      if ((e2 >> o) & 1u) cur_e = p;
    }
  }
  // what is kept, by side and by "rank inside the own part >= size of the other part"
  const bool a_ge = g.op != THRUST_AMD_SET_INTERSECTION;                                  // A, rank >= |B part|
  const bool a_lt = g.op == THRUST_AMD_SET_INTERSECTION || g.op == THRUST_AMD_SET_UNION;  // A, rank <  |B part|
  const bool b_ge = g.op == THRUST_AMD_SET_SYMMETRIC_DIFFERENCE || g.op == THRUST_AMD_SET_UNION;
  uint32_t keep = 0;
  {
    uint32_t cur_h = (uint32_t)(fwd_in >> 32);  // p + 1 of the last run start at or before the element
    uint32_t cur_e = (uint32_t)fwd_in;          // p + 1 of the last B-part start at or before it
#pragma unroll
    for (int o = 0; o < SET_ITEMS; ++o) {
      const uint32_t p = run0 + o;
      if ((head >> o) & 1u) cur_h = p + 1;
      if ((e2 >> o) & 1u) cur_e = p + 1;
      const bool bo = (is_b >> o) & 1u;
      // an interior run starts inside the tile (cur_h >= 1); for a B, the run's first B is at or before p
      const uint32_t n_b = (o & 1) ? (b_after[o / 2] >> 16) : (b_after[o / 2] & 0xffffu);
      const uint32_t own_start = (bo ? cur_e : cur_h) - 1u;
      const uint32_t other = bo ? cur_e - cur_h : n_b;
      const bool ge_local = p - own_start >= other;
      const bool ge_first = p >= (bo ? thr_b0 : thr_a0);
      const bool ge_next = p >= (bo ? thr_b1 : thr_a1);
      const bool ge = (p < first_end) ? ge_first : ((tail_continues && p >= last_start) ? ge_next : ge_local);
      const bool kp = bo ? (b_ge && ge) : (ge ? a_ge : a_lt);
      keep |= (uint32_t)kp << o;
    }
    keep &= live;
  }

  // ---- ranks inside the tile, then the tile's place in the output
  uint32_t tile_cnt = 0;
  __syncthreads();  // s_scan32 is fresh, but s_keys is about to be overwritten: all merges are done
  const uint32_t mine = __builtin_popcount(keep);
  const uint32_t excl = set_block_exclusive<SET_WAVES, uint32_t>(mine, OpPlus{}, 0u, s_scan32, &tile_cnt);

  constexpr int W = TileWords<uint64_t>::W;
  uint64_t* my_slot = g.status + (size_t)tile * W;
  if (threadIdx.x < WAVE) {
    const int lane = threadIdx.x;
    uint64_t before = 0;
    if (tile == 0) {
      if (lane == 0) tile_publish<uint64_t>(my_slot, TS_INCLUSIVE, (uint64_t)tile_cnt);
    } else {
      if (lane == 0) tile_publish<uint64_t>(my_slot, TS_PARTIAL, (uint64_t)tile_cnt);
      before = tile_lookback<uint64_t>(g.status, (uint32_t)tile, OpPlus{}, (uint64_t)0);
      if (lane == 0) tile_publish<uint64_t>(my_slot, TS_INCLUSIVE, before + tile_cnt);
    }
    if (lane == 0) {
      s_base = before;
      if (d1 == total) *g.d_num = before + tile_cnt;
    }
  }

  // ---- compaction through LDS (the staging area is free: every lane has merged)
  {
    uint32_t r = excl;
#pragma unroll
    for (int o = 0; o < SET_ITEMS; ++o) {
      if ((keep >> o) & 1u) {
        s_keys[r] = k[o];
        if constexpr (HAS_VALUES) s_src[r] = (uint16_t)slot[o];
        ++r;
      }
    }
  }
  __syncthreads();
  const uint64_t base = s_base;
#pragma unroll
  for (int q = 0; q < SET_ITEMS; ++q) {
    const uint32_t e = q * SET_BLOCK + threadIdx.x;
    if (e < tile_cnt) g.out[base + e] = s_keys[e];
  }
  if constexpr (HAS_VALUES) {
    // values: the two sub-ranges are staged like the keys were (A's part, then B's, so a
    // key's staging slot is its value's), then gathered by slot in output order
    const bool keeps_b = g.op == THRUST_AMD_SET_SYMMETRIC_DIFFERENCE || g.op == THRUST_AMD_SET_UNION;
    __syncthreads();  // the compacted keys have been read
    {
      V in[SET_ITEMS];
#pragma unroll
      for (int q = 0; q < SET_ITEMS; ++q) {
        const uint32_t e = q * SET_BLOCK + threadIdx.x;
        in[q] = (e < ca) ? g.va[a0 + e] : (keeps_b && e < count) ? g.vb[b0 + (e - ca)] : V{};
      }
#pragma unroll
      for (int q = 0; q < SET_ITEMS; ++q) s_vals[q * SET_BLOCK + threadIdx.x] = in[q];
    }
    __syncthreads();
#pragma unroll
    for (int q = 0; q < SET_ITEMS; ++q) {
      const uint32_t e = q * SET_BLOCK + threadIdx.x;
      if (e < tile_cnt) g.vout[base + e] = s_vals[s_src[e]];  // s_src[e] < count
    }
  }
}

// Where the pieces of one call's temporary storage lie.
template <typename T, typename V, bool HAS_VALUES>
struct SetTemp {
  using Shape = SetShape<T, V, HAS_VALUES>;
  uint64_t tiles;
  size_t off_ticket, off_split, off_run, off_key, off_status, total;
  explicit SetTemp(uint64_t elements) : tiles((elements + Shape::TILE - 1) / Shape::TILE) {
    TempLayout lay;
    off_ticket = lay.add(sizeof(uint32_t));
    off_split = lay.add((size_t)(tiles + 1) * sizeof(uint64_t));
    off_run = lay.add((size_t)(tiles + 1) * 3 * sizeof(uint64_t));
    off_key = lay.add((size_t)(tiles + 1) * sizeof(T));
    off_status = lay.add((size_t)tiles * TileWords<uint64_t>::W * sizeof(uint64_t));
    total = lay.total;
  }
};

// The three kernels of one set operation; temp holds SetTemp<T, V, HAS_VALUES>(na + nb).total
// bytes, *d_num receives the size of the result.
template <typename T, typename V, bool HAS_VALUES, typename Comp>
inline int set_launch(char* temp, int op, const T* a, uint64_t na, const T* b, uint64_t nb, const V* va, const V* vb,
                      T* out, V* vout, uint64_t* d_num, Comp comp, hipStream_t stream) {
  using Shape = SetShape<T, V, HAS_VALUES>;
  const uint64_t total = na + nb;
  const SetTemp<T, V, HAS_VALUES> lay(total);
  const uint64_t tiles = lay.tiles;
  if (tiles > 0x7fffffffull) return (int)hipErrorInvalidValue;
  uint32_t* ticket = reinterpret_cast<uint32_t*>(temp + lay.off_ticket);
  uint64_t* split = reinterpret_cast<uint64_t*>(temp + lay.off_split);
  uint64_t* run = reinterpret_cast<uint64_t*>(temp + lay.off_run);
  T* key = reinterpret_cast<T*>(temp + lay.off_key);
  uint64_t* status = reinterpret_cast<uint64_t*>(temp + lay.off_status);
  const uint64_t words = tiles * TileWords<uint64_t>::W;
  THRUST_AMD_KERNEL_LAUNCH("set_init", stream, set_init_kernel<0>, dim3((uint32_t)((words + 255) / 256 + 1)), dim3(256),
                           status, words, ticket, d_num);
  hipError_t e = hipPeekAtLastError();
  if (e != hipSuccess) return (int)e;
  if (total == 0) return 0;
  THRUST_AMD_KERNEL_LAUNCH("set_partition", stream, (set_partition_kernel<T, Comp>),
                           dim3((uint32_t)((tiles + 1 + 255) / 256)), dim3(256), a, na, b, nb, tiles,
                           (uint32_t)Shape::TILE, comp, split, run, key);
  e = hipPeekAtLastError();
  if (e != hipSuccess) return (int)e;
  SetArgs<T, V, HAS_VALUES, Comp> g{a,   b,      va,     vb,    out,   vout, na, nb,  (const uint64_t*)split, (const uint64_t*)run,
                                    key, status, ticket, d_num, tiles, op,   comp};
  THRUST_AMD_KERNEL_LAUNCH("set_operation", stream, (set_op_kernel<T, V, HAS_VALUES, Comp>), dim3((uint32_t)tiles),
                           dim3(Shape::BLOCK), g);
  return (int)hipPeekAtLastError();
}

}  // namespace setops
}  // namespace hip
}  // namespace system
}  // namespace thrust
