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
// the run starts, where its B part starts and where it ends.  An element of the part that
// comes second in the run has everything it needs before it on the path; an element of the
// first part needs to know how many elements of the second part follow.  Difference and
// intersection only ever keep elements of A, so for them the two ranges change places (ties
// go to B, a run is B_0 .. B_{n-1} A_0 .. A_{m-1}) and nothing has to look ahead; only the
// symmetric difference decides elements of both parts and pays for the look ahead.  Below,
// "A" and "B" name the ranges in the order the kernels receive them.
//
//   partition  one thread per tile boundary: the merge-path split, and the three
//              positions (searched outward from the split) of the run that
//              contains the first element of the tile -- the only run of a tile that can
//              start before it, and, read from the next boundary, the only one that can
//              end after it
//   tile       stages its two sub-ranges in LDS and merges them serially per lane as
//              the merge kernel does; head flags on the merged order (a lane's predecessor
//              key is the later of the two elements before its merge-path split); the last run
//              start and B-part start before every lane, and the next ones after it, travel
//              as pairs of 16-bit positions through one forward and one backward max-scan
//              behind a single barrier (the backward one only for the symmetric difference);
//              each lane then walks its 16 elements once per side that the operation
//              decides (A: rank against the B elements that follow in
//              the run; B: position against a threshold fixed where the B part starts), in
//              lane-relative positions, collecting the outcomes as sign bits; keep flags ->
//              ranks -> decoupled look-back over the tiles' counts (dynamic tickets) ->
//              compaction through LDS -> coalesced stores; values are gathered from the
//              range their key came from
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
  static constexpr int WAVES_PER_SIMD = ITEM > 4 ? 3 : (HAS_VALUES ? 4 : 8);
};

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
  // first index whose element is not before x / is after x, in each range: the run of x lies
  // around the split, a few elements long unless the input repeats itself
  const uint64_t lb_a = nearby_partition_point(0, na, as, [&](uint64_t i) { return comp(a[i], x); });
  const uint64_t ub_a = nearby_partition_point(lb_a, na, as, [&](uint64_t i) { return !comp(x, a[i]); });
  const uint64_t lb_b = nearby_partition_point(0, nb, bs, [&](uint64_t i) { return comp(b[i], x); });
  const uint64_t ub_b = nearby_partition_point(lb_b, nb, bs, [&](uint64_t i) { return !comp(x, b[i]); });
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

// Two tile-local positions that travel through a max-scan together, 16 bits each.
struct OpMaxPair16 {
  THRUST_AMD_DEVICE uint32_t operator()(uint32_t x, uint32_t y) const {
    typedef unsigned short pair16 __attribute__((ext_vector_type(2)));
    pair16 a, b;
    __builtin_memcpy(&a, &x, 4);
    __builtin_memcpy(&b, &y, 4);
    const pair16 m = __builtin_elementwise_max(a, b);
    uint32_t r;
    __builtin_memcpy(&r, &m, 4);
    return r;
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

// Two scans of position pairs behind one barrier: `before` = the fold of `fwd` over the
// threads before this one, `after` = the fold of `bwd` over the threads after it (0 unless
// `backward`, which is the same for the whole workgroup), `all` = the fold of `fwd` over the
// workgroup.  0 is the identity.
template <int WAVES>
THRUST_AMD_DEVICE void set_block_both_ways(uint32_t fwd, uint32_t bwd, bool backward, uint32_t* buf_fwd,
                                           uint32_t* buf_bwd, uint32_t& before, uint32_t& after, uint32_t& all) {
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const OpMaxPair16 op;
  const int mirror = (WAVE - 1 - lane) * 4;
  const uint32_t incl_f = wave_inclusive_scan(fwd, op, 0u);
  if (lane == WAVE - 1) buf_fwd[wave] = incl_f;
  const uint32_t excl_f = dpp_move<0x138 /* wave_shr:1 */>(0u, incl_f);
  uint32_t excl_b = 0;
  if (backward) {
    const uint32_t incl_b = wave_inclusive_scan((uint32_t)__builtin_amdgcn_ds_bpermute(mirror, (int)bwd), op, 0u);
    if (lane == WAVE - 1) buf_bwd[wave] = incl_b;
    excl_b = (uint32_t)__builtin_amdgcn_ds_bpermute(mirror, (int)dpp_move<0x138 /* wave_shr:1 */>(0u, incl_b));
  }
  __syncthreads();
  uint32_t prefix = 0, total = 0, suffix = 0;
#pragma unroll
  for (int w = 0; w < WAVES; ++w) {
    if (w == wave) prefix = total;
    total = op(total, buf_fwd[w]);
  }
  if (backward) {
#pragma unroll
    for (int w = 0; w < WAVES; ++w)
      if (w > wave) suffix = op(suffix, buf_bwd[w]);
  }
  before = op(prefix, excl_f);
  after = op(suffix, excl_b);
  all = total;
}

// all ones when bit `o` of `bits` is set, else zero
THRUST_AMD_DEVICE int32_t set_bit_mask(uint32_t bits, int o) { return (int32_t)(bits << (31 - o)) >> 31; }
// `yes` where the mask is all ones, `no` where it is zero
THRUST_AMD_DEVICE int32_t set_pick(int32_t mask, int32_t yes, int32_t no) { return (yes & mask) | (no & ~mask); }

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
  static_assert(SET_TILE <= 0x7fff && SET_ITEMS == 16, "positions travel in 16 bits, flags in 16-bit masks");
  // one buffer for the staged keys, the compacted keys and (later) the staged values
  // (lanes past the end of a short tile read up to SET_ITEMS slots past it)
  __shared__ __attribute__((aligned(16))) unsigned char s_raw[(size_t)(SET_TILE + SET_ITEMS) * Shape::ITEM];
  T* s_keys = reinterpret_cast<T*>(s_raw);
  V* s_vals = reinterpret_cast<V*>(s_raw);
  __shared__ uint16_t s_src[HAS_VALUES ? SET_TILE : 1];
  __shared__ uint32_t s_fwd[SET_WAVES];
  __shared__ uint32_t s_bwd[SET_WAVES];
  __shared__ uint32_t s_scan32[SET_WAVES];
  __shared__ uint32_t s_tile;
  __shared__ uint64_t s_base;

  Comp& comp = g.comp;
  if (threadIdx.x == 0) s_tile = atomicAdd(g.ticket, 1u);
  __syncthreads();
  // the ticket and what follows from it are the same for the whole workgroup: scalar registers
  const uint64_t tile = (uint32_t)__builtin_amdgcn_readfirstlane((int)s_tile);
  const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x / WAVE));
  const uint32_t lane = threadIdx.x % WAVE;
  const uint64_t total = g.na + g.nb;
  const uint64_t d0 = tile * SET_TILE;
  const uint64_t d1 = (d0 + SET_TILE < total) ? d0 + SET_TILE : total;
  const uint64_t a0 = g.split[tile], a1 = g.split[tile + 1];
  const uint64_t b0 = d0 - a0, b1 = d1 - a1;
  const uint32_t ca = (uint32_t)(a1 - a0), cb = (uint32_t)(b1 - b0);
  const uint32_t count = ca + cb;  // == d1 - d0, 1 .. SET_TILE

  // The run the tile starts in is the only one that can begin before the tile.  With rs / rm /
  // re the merged positions where it starts, where its B part starts and where it ends, its
  // element at merged position P has rank P - rs >= (re - rm) [A] or P - rm >= (rm - rs) [B]
  // exactly when its tile-local position is at or past a threshold (used when that run
  // covers the whole tile; otherwise its start and its B part seed the lanes' states below).
  constexpr uint32_t FAR = 4u * SET_TILE;  // counts at or above this decide like any larger one
  const bool f1_valid = d1 < total;
  uint32_t thr_a0, thr_b0;
  int32_t first_start;   // local position where the tile's first run starts (<= 0), bounded below
  bool first_b_before;   // its B part starts before the tile
  {
    const uint64_t rs = g.run[3 * tile], rm = g.run[3 * tile + 1], re = g.run[3 * tile + 2];
    auto local_threshold = [&](uint64_t global_pos) -> uint32_t {
      if (global_pos <= d0) return 0u;
      const uint64_t rel = global_pos - d0;
      return rel > (uint64_t)SET_TILE ? (uint32_t)SET_TILE + 1u : (uint32_t)rel;
    };
    thr_a0 = local_threshold(rs + (re - rm));
    thr_b0 = local_threshold(rm + (rm - rs));
    const uint64_t back = d0 - rs;
    first_start = -(int32_t)(back < (uint64_t)SET_TILE + 1u ? (uint32_t)back : (uint32_t)SET_TILE + 1u);
    first_b_before = rm < d0;
  }

  // Only the symmetric difference decides elements of the first range (their rank against the
  // elements of the second range, which follow them in the run); elements of the second range
  // are decided by every operation, against what came before them.
  const bool need_a = g.op == THRUST_AMD_SET_SYMMETRIC_DIFFERENCE;
  constexpr bool need_b = true;

  // ---- stage the keys: A's part first, then B's
  stage_two_parts<SET_BLOCK, SET_ITEMS>(g.a + a0, g.b + b0, ca, count, s_keys);
  __syncthreads();

  // ---- this lane's start on the path, then a serial merge of ITEMS elements
  const uint32_t run0 = threadIdx.x * SET_ITEMS;
  const uint32_t diag = run0 < count ? run0 : count;
  const uint32_t i = merge_path_in_tile(s_keys, ca, count, diag, comp);
  const uint32_t j = ca + (diag - i);
  // the element before this lane's first one is the later of the two last ones taken so far (B after A on ties)
  bool prev_is_b;
  T prev_key;
  {
    const T last_a = s_keys[i > 0 ? i - 1 : 0], last_b = s_keys[j > ca ? j - 1 : ca];
    prev_is_b = (j > ca) && (i == 0 || !comp(last_b, last_a));
    prev_key = prev_is_b ? last_b : last_a;
    if (threadIdx.x == 0) prev_is_b = first_b_before;  // the element before the tile, if it belongs to the same run
  }
  T k[SET_ITEMS];
  uint32_t slot[SET_ITEMS];
  uint32_t is_b = 0;  // bit o: merged element o of this lane comes from B
  merge_steps<SET_ITEMS>(s_keys, i, j, ca, count, comp, [&](int o, const T& x, uint32_t from, bool take_b) {
    k[o] = x;
    slot[o] = from;
    is_b |= (uint32_t)take_b << o;
  });
  // valid elements of this lane: merged positions run0 + o < count
  const uint32_t live = (run0 >= count) ? 0u : ((count - run0 >= (uint32_t)SET_ITEMS) ? 0xffffu : ((1u << (count - run0)) - 1u));

  // B elements of the tile's last run that lie in later tiles (the last merged key is the later
  // of the two parts' last keys; only its equivalence class matters)
  uint32_t tail_b = 0;
  if (need_a && f1_valid) {
    const T last_a = s_keys[ca ? ca - 1 : 0], last_b = s_keys[count - 1];
    const T last = (cb == 0) ? last_a : (ca == 0) ? last_b : (comp(last_b, last_a) ? last_a : last_b);
    const T f1_key = g.key[tile + 1];
    if (!comp(last, f1_key)) {
      const uint64_t rm = g.run[3 * (tile + 1) + 1], re = g.run[3 * (tile + 1) + 2];
      const uint64_t beyond = re - (rm > d1 ? rm : d1);
      tail_b = beyond < (uint64_t)FAR ? (uint32_t)beyond : FAR;
    }
  }

  // ---- head flags on the merged order: bit o set when valid element o starts a run (local
  // position 0 never counts: the first run's start is known from the partition); e2: first
  // B of a run, i.e. a B whose predecessor is an A or that starts a run
  uint32_t head = 0;
  {
    T prev = (threadIdx.x > 0) ? prev_key : k[0];
#pragma unroll
    for (int o = 0; o < SET_ITEMS; ++o) {
      head |= (uint32_t)comp(prev, k[o]) << o;
      prev = k[o];
    }
    head &= live;
  }
  const uint32_t prev_b_bits = (is_b << 1) | (uint32_t)prev_is_b;
  const uint32_t e2 = is_b & (head | ~prev_b_bits) & live;

  // ---- for every lane: the last run start and B-part start before its elements (positions
  // + 1, 0 = none) and the next ones after them (SET_TILE - position, 0 = none)
  uint32_t fwd_in, bwd_in, fwd_all;
  {
    const uint32_t last_h = head ? run0 + (31 - __builtin_clz(head)) + 1 : 0u;
    const uint32_t last_e2 = e2 ? run0 + (31 - __builtin_clz(e2)) + 1 : 0u;
    const uint32_t first_h = head ? SET_TILE - (run0 + __builtin_ctz(head)) : 0u;
    const uint32_t first_e2 = e2 ? SET_TILE - (run0 + __builtin_ctz(e2)) : 0u;
    set_block_both_ways<SET_WAVES>((last_h << 16) | last_e2, (first_h << 16) | first_e2, need_a, s_fwd, s_bwd, fwd_in,
                                   bwd_in, fwd_all);
  }

  // ---- decide every element: lt_a / lt_b, bit o = element o (of A / of B) has a rank inside
  // its own part of the run that is below the size of the other part.  Positions are
  // relative to the lane's first element from here on, and signed.
  uint32_t lt_a = 0, lt_b = 0;
  if ((fwd_all >> 16) == 0) {
    // no run starts inside the tile: the first run covers it, and the thresholds decide
    auto below = [&](uint32_t thr) -> uint32_t {
      const uint32_t c = thr > run0 ? (thr - run0 < (uint32_t)SET_ITEMS ? thr - run0 : (uint32_t)SET_ITEMS) : 0u;
      return (1u << c) - 1u;
    };
    lt_a = below(thr_a0);
    lt_b = below(thr_b0);
  } else {
    const uint32_t h_in = fwd_in >> 16, e_in = fwd_in & 0xffffu;
    const int32_t start = h_in ? (int32_t)h_in - 1 - (int32_t)run0 : first_start - (int32_t)run0;
    // Most elements of B need no positions: one that starts a run faces no element of A and is
    // not below; one that follows an element of A in its run has rank 0 and is below; one that
    // follows an element of B that is not below is not below either.  Only an element of B after
    // an element of B that may be below (one that does not start the run) has to count, and a wave
    // without such an element decides with three bit operations.  (The element before a wave's
    // first one counts as one that may be below.)
    const uint32_t head_all = head | (uint32_t)(threadIdx.x == 0 && first_start == 0);  // the tile's first element too
    const uint32_t head_before =
        (head_all << 1) | (lane == 0 ? 0u : dpp_move<0x138 /* wave_shr:1 */>(0u, (head_all >> (SET_ITEMS - 1)) & 1u));
    const uint32_t counts = is_b & ~head_all & prev_b_bits & ~head_before & live;
    if (__builtin_amdgcn_ballot_w64(counts != 0) == 0) {
      lt_b = is_b & ~head_all & ~prev_b_bits;
    } else {
      // an element of B at position p, in a run that starts at s and whose B part starts at m,
      // has rank p - m and faces m - s elements of A: below exactly when p < 2m - s
      int32_t s = start;
      int32_t tb = (e_in != 0 && e_in >= h_in) ? 2 * ((int32_t)e_in - 1 - (int32_t)run0) - s
                   : (h_in == 0 && first_b_before) ? (int32_t)thr_b0 - (int32_t)run0
                                                   : 0x10000;  // no B of this run yet: the first one sets it
      uint32_t acc = 0;
#pragma unroll
      for (int o = 0; o < SET_ITEMS; ++o) {
        s = set_pick(set_bit_mask(head, o), o, s);
        tb = set_pick(set_bit_mask(e2, o), 2 * o - s, tb);
        acc = __builtin_amdgcn_alignbit(acc, (uint32_t)(o - tb), 31);  // shifts the sign in: o < tb
      }
      lt_b = __builtin_bitreverse32(acc) >> 16;
    }
    if (need_a) {
      // an element of A at position p has rank p - s and faces all B elements of its run, which
      // come after it: those in this lane, and after the lane those up to the next run start
      const uint32_t nh_m = bwd_in >> 16, ne_m = bwd_in & 0xffffu;
      const uint32_t end_l = run0 + SET_ITEMS < count ? run0 + SET_ITEMS : count;
      const bool last_is_b = (is_b & live) > (live >> 1);
      uint32_t nb;
      if (nh_m) nb = last_is_b ? (SET_TILE - nh_m) - end_l : (ne_m > nh_m ? ne_m - nh_m : 0u);
      else nb = (last_is_b ? count - end_l : (ne_m ? count - (SET_TILE - ne_m) : 0u)) + tail_b;
      uint32_t facing[SET_ITEMS];
      const uint32_t not_head = ~head;
#pragma unroll
      for (int o = SET_ITEMS - 1; o >= 0; --o) {
        facing[o] = nb;
        nb += (is_b >> o) & 1u;
        nb &= (uint32_t)set_bit_mask(not_head, o);
      }
      int32_t s = start;
      uint32_t acc = 0;
#pragma unroll
      for (int o = 0; o < SET_ITEMS; ++o) {
        s = set_pick(set_bit_mask(head, o), o, s);
        acc = __builtin_amdgcn_alignbit(acc, (uint32_t)((o - s) - (int32_t)facing[o]), 31);  // rank < facing
      }
      lt_a = __builtin_bitreverse32(acc) >> 16;
    }
  }
  // union: all of the first range, of the second those at or above; symmetric difference: of both
  // those at or above; difference and intersection (whose first range is the caller's second):
  // nothing of the first range, of the second those at or above / those below
  const uint32_t keep_a = g.op == THRUST_AMD_SET_UNION ? ~0u : (need_a ? ~lt_a : 0u);
  const uint32_t keep_b = g.op == THRUST_AMD_SET_INTERSECTION ? lt_b : ~lt_b;
  const uint32_t keep = ((~is_b & keep_a) | (is_b & keep_b)) & live;

  // ---- ranks inside the tile, then the tile's place in the output
  uint32_t tile_cnt_v = 0;
  const uint32_t mine = __builtin_popcount(keep);
  const uint32_t excl = set_block_exclusive<SET_WAVES, uint32_t>(mine, OpPlus{}, 0u, s_scan32, &tile_cnt_v);
  const uint32_t tile_cnt = (uint32_t)__builtin_amdgcn_readfirstlane((int)tile_cnt_v);

  constexpr int W = TileWords<uint64_t>::W;
  uint64_t* my_slot = g.status + (size_t)tile * W;
  if (threadIdx.x < WAVE) {
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

  // ---- compaction through LDS (the staging area is free: every lane has merged, two barriers ago)
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
  uint64_t base;
  {
    const uint64_t b64 = s_base;
    base = ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(b64 >> 32)) << 32) |
           (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)b64);
  }
  {
    T* dst = g.out + base;
#pragma unroll
    for (int q = 0; q < SET_ITEMS; ++q) {
      const uint32_t row = (uint32_t)q * SET_BLOCK + wave * WAVE;
      if (row + WAVE <= tile_cnt) dst[row + lane] = s_keys[row + lane];
      else if (row + lane < tile_cnt) dst[row + lane] = s_keys[row + lane];
    }
  }
  if constexpr (HAS_VALUES) {
    // values: the two sub-ranges are staged like the keys were (A's part, then B's, so a
    // key's staging slot is its value's), then gathered by slot in output order
    __syncthreads();  // the compacted keys have been read
    // (the first range's values are only read by the operations that can keep one of its elements)
    if (g.op == THRUST_AMD_SET_UNION || g.op == THRUST_AMD_SET_SYMMETRIC_DIFFERENCE) {
      stage_two_parts<SET_BLOCK, SET_ITEMS>(g.va + a0, g.vb + b0, ca, count, s_vals);
    } else {
      const V* const second = g.vb + b0;
      V in[SET_ITEMS];
#pragma unroll
      for (int q = 0; q < SET_ITEMS; ++q) {
        const uint32_t e = (uint32_t)q * SET_BLOCK + threadIdx.x;
        if (e >= ca && e < count) in[q] = second[e - ca];
      }
#pragma unroll
      for (int q = 0; q < SET_ITEMS; ++q) {
        const uint32_t e = (uint32_t)q * SET_BLOCK + threadIdx.x;
        if (e >= ca && e < count) s_vals[e] = in[q];
      }
    }
    __syncthreads();
    V* dst = g.vout + base;
#pragma unroll
    for (int q = 0; q < SET_ITEMS; ++q) {
      const uint32_t row = (uint32_t)q * SET_BLOCK + wave * WAVE;
      if (row + WAVE <= tile_cnt) dst[row + lane] = s_vals[s_src[row + lane]];
      else if (row + lane < tile_cnt) dst[row + lane] = s_vals[s_src[row + lane]];  // s_src[e] < count
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
  // Difference and intersection keep elements of A only, each decided by its rank against the
  // number of equivalent elements of B.  The kernel decides the elements of its second range
  // from what precedes them on the merge path, so for these two the ranges change places: ties
  // then go to B, and an element of A has all of its run's elements of B before it.
  if (op == THRUST_AMD_SET_DIFFERENCE || op == THRUST_AMD_SET_INTERSECTION) {
    const T* const ta = a;
    a = b;
    b = ta;
    const V* const tv = va;
    va = vb;
    vb = tv;
    const uint64_t tn = na;
    na = nb;
    nb = tn;
  }
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
