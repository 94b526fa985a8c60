// thrust_amd_sort_keys / thrust_amd_sort_pairs: onesweep least-significant-digit radix sort.
//
//   init       zeroes the digit histograms, the per-pass tile descriptors and tickets
//   histogram  one read of the keys builds the 256-bin histogram of EVERY 8-bit digit
//   scan       exclusive scan of each histogram -> global digit offsets; a digit whose one
//              bin holds all n keys is marked "skip" (the reference's sequential radix
//              sort does the same, thrust/system/detail/sequential/stable_radix_sort.inl:
//              264-283), and the ping-pong source of every pass is derived from that
//   pass x P   chained digit-binning pass ("onesweep"): a tile ranks its keys by digit,
//              learns the global offset of each of its 256 digit runs by decoupled
//              look-back over the tiles before it, and scatters keys (and values)
//   copy-back  only if an odd number of passes ran
//
// Ranking inside a tile uses the wave64 match pattern: for each of the 8 digit bits one
// ballot, folded into a 64-bit peer mask with v_bitop3; rank = wave-private LDS counter
// + number of peers in lower lanes (v_mbcnt accumulates onto the counter's value).  Lanes hold keys wave-striped (lane l of wave w holds
// keys l, 64+l, ... of the wave's span), so (round, lane) order is memory order and the
// pass is stable.  Keys and values are then exchanged through LDS so that global stores
// are contiguous per digit run.
//
// Tile order is a dynamic ticket, so the look-back only waits for tiles that have
// started: one ticket counter per class of blockIdx % 8, so that neighbouring tiles run on
// the same XCD (sort_tickets.hpp).  Tile descriptors are one word per (tile, digit): 2 status bits above a count,
// 32-bit words for n < 2^30 keys and 64-bit words up to the limit of 2^32 - 1 keys per call
// (positions and histogram counts are 32-bit).
//
// Algorithmic HBM traffic for K-byte keys, V-byte values, P = K passes:
// K*n (histogram) + P * 2*(K+V)*n.  Replaces cub::DeviceRadixSort as called from
// thrust/system/cuda/detail/sort.h:1326-1508.
#include "common.hpp"
#include "dispatch.hpp"
#include "launch.hpp"
#include "sort_tickets.hpp"

namespace ta {

constexpr int RADIX_BITS = 8;
constexpr int RADIX_SIZE = 1 << RADIX_BITS;
constexpr int MAX_PASSES = 8;
constexpr uint64_t SORT_MAX_N = (1ull << 32) - 1;       // positions and counts are 32-bit
constexpr uint64_t SORT_MAX_N_NARROW = (1ull << 30) - 1;  // ... and fit 30 bits up to here

// Tile descriptor word: 2 status bits above a count.  32-bit words (30-bit counts) serve
// sorts of fewer than 2^30 keys, 64-bit words the larger ones.
template <typename D>
struct Descriptor {
  static constexpr int SHIFT = (int)sizeof(D) * 8 - 2;
  static constexpr D VALUE_MASK = ((D)1 << SHIFT) - 1;
  static constexpr D PARTIAL = (D)1 << SHIFT;
  static constexpr D INCLUSIVE = (D)2 << SHIFT;
};

// Key <-> radix encoding, decided at run time (uniform across the grid).
//   sign:   sign bit for signed integers and floats, else 0
//   fmask:  all ones for floating point, else 0
//   dmask:  all ones for descending order, else 0
template <typename K>
struct KeyCodec {
  K sign, fmask, dmask;
  uint32_t plain;  // all three masks are zero: encode/decode are the identity
  TA_DEVICE K encode(K k) const {
    using SK = typename std::make_signed<K>::type;
    const K neg = (K)((SK)k >> (sizeof(K) * 8 - 1));
    return k ^ ((neg & fmask) | sign) ^ dmask;
  }
  TA_DEVICE K decode(K e) const {
    using SK = typename std::make_signed<K>::type;
    e ^= dmask;
    const K pos = (K)((SK)e >> (sizeof(K) * 8 - 1));
    return e ^ ((~pos & fmask) | sign);
  }
};

struct SortCtl {
  uint32_t skip[MAX_PASSES];     // pass moves nothing
  uint32_t src_alt[MAX_PASSES];  // pass reads the alternate buffer
  uint32_t final_in_alt;         // result sits in the alternate buffer after the last pass
  uint32_t gave_up;              // a tile stopped waiting for its predecessors (see LOOKBACK_SPIN_LIMIT)
};

constexpr uint32_t TICKET_WORDS = MAX_PASSES * TICKET_CLASSES * TICKET_STRIDE;

// A tile waits for its predecessors' counts in a loop.  Every predecessor is taken by a running
// workgroup as long as every class keeps receiving its workgroups while slots are free -- which
// holds when workgroups are bound to XCDs in turn, and when they are dispatched in order to at
// least 64 slots.  Should neither hold, a tile that has polled this often stops waiting: it
// uses what it has summed so far (its positions stay inside the array: a prefix can only be too
// small), sets SortCtl::gave_up, and every tile that sees the flag does the same, so the
// kernel ends -- with keys out of order -- instead of hanging.
constexpr uint32_t LOOKBACK_SPIN_LIMIT = 1u << 21;

struct SortGeometry {
  int passes;
  int begin_bit;
  int end_bit;
};

// ------------------------------------------------------------------ init
__global__ __launch_bounds__(256) void sort_init_kernel(uint32_t* __restrict__ words, uint64_t count) {
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += stride)
    words[i] = 0;
}

// ------------------------------------------------------------------ histogram
// One workgroup per CU with up to 128 KiB of LDS: every bin exists in COPIES copies and
// lane l only ever touches copy l % COPIES, so with 32 copies the 64 lanes of an LDS
// atomic fall on 32 distinct banks whatever the digits are (random digits on a single
// copy serialise about five-fold on bank conflicts).  Keys are read with 16-byte loads;
// their order does not matter here.
// WHOLE_BYTES: the keys need no encoding and the sorted bits are NP whole bytes starting
// at bit 0 (the usual full-range sort of unsigned keys), so every digit is a bit-field
// extract at a constant position.
constexpr int HIST_BLOCK = 1024;
constexpr int HIST_UNROLL = 4;  // 16-byte vectors in flight per lane

template <typename K, int NP, bool WHOLE_BYTES>
__global__ __launch_bounds__(HIST_BLOCK) void sort_histogram_kernel(const K* __restrict__ keys,
                                                                     uint64_t n, KeyCodec<K> codec,
                                                                     SortGeometry geo,
                                                                     uint32_t* __restrict__ hist) {
  constexpr int COPIES = NP <= 4 ? 32 : 16;
  constexpr int BINS = NP * RADIX_SIZE;
  constexpr int VEC = Vec16<K>::N;
  __shared__ uint32_t s_hist[BINS * COPIES];
  for (int i = threadIdx.x; i < BINS * COPIES; i += HIST_BLOCK) s_hist[i] = 0;
  __syncthreads();
  uint32_t* my_copy = s_hist + (threadIdx.x % COPIES);

  auto count = [&](K k) {
    const K e = (WHOLE_BYTES || codec.plain) ? k : codec.encode(k);
#pragma unroll
    for (int p = 0; p < NP; ++p) {
      const int lo = WHOLE_BYTES ? p * RADIX_BITS : geo.begin_bit + p * RADIX_BITS;
      const int nb = (WHOLE_BYTES || p < NP - 1) ? RADIX_BITS : (geo.end_bit - lo);
      const uint32_t d = (uint32_t)(e >> lo) & ((1u << nb) - 1u);
      __hip_atomic_fetch_add(my_copy + (p * RADIX_SIZE + d) * COPIES, 1u, __ATOMIC_RELAXED,
                             __HIP_MEMORY_SCOPE_WORKGROUP);
    }
  };

  // head: elements before the first 16-byte boundary; tail: what the vectors leave over
  const uint64_t mis = (reinterpret_cast<uintptr_t>(keys) & 15u) / sizeof(K);
  const uint64_t head = mis ? ((VEC - mis) < n ? (VEC - mis) : n) : 0;
  const uint64_t vecs = (n - head) / VEC;
  const uint64_t tail_begin = head + vecs * VEC;
  if (blockIdx.x == 0) {
    if (threadIdx.x < head) count(keys[threadIdx.x]);
    if (tail_begin + threadIdx.x < n) count(keys[tail_begin + threadIdx.x]);
  }
  const Vec16<K>* body = reinterpret_cast<const Vec16<K>*>(keys + head);
  constexpr uint64_t TILE_VECS = (uint64_t)HIST_BLOCK * HIST_UNROLL;
  // Whole tiles: no predicates, and the next tile's vectors are in flight while this
  // tile's are counted (two register buffers in turn; the loop body always loads, so
  // the waits before counting only cover the older buffer).
  const uint64_t whole_tiles = vecs / TILE_VECS;
  const uint64_t step = gridDim.x;
  uint64_t tile = blockIdx.x;
  Vec16<K> buf_a[HIST_UNROLL], buf_b[HIST_UNROLL];
  auto load_tile = [&](Vec16<K>(&x)[HIST_UNROLL], uint64_t t) {
#pragma unroll
    for (int u = 0; u < HIST_UNROLL; ++u) x[u] = body[t * TILE_VECS + threadIdx.x + (uint64_t)u * HIST_BLOCK];
  };
  auto count_tile = [&](const Vec16<K>(&x)[HIST_UNROLL]) {
#pragma unroll
    for (int u = 0; u < HIST_UNROLL; ++u) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) count(x[u].v[i]);
    }
  };
  if (tile < whole_tiles) load_tile(buf_a, tile);
  while (tile + 2 * step < whole_tiles) {
    load_tile(buf_b, tile + step);
    count_tile(buf_a);
    load_tile(buf_a, tile + 2 * step);
    count_tile(buf_b);
    tile += 2 * step;
  }
  if (tile < whole_tiles) {
    if (tile + step < whole_tiles) {
      load_tile(buf_b, tile + step);
      count_tile(buf_a);
      count_tile(buf_b);
    } else {
      count_tile(buf_a);
    }
  }
  // the ragged tile after them, if any, goes to the workgroup whose turn it would be
  if (whole_tiles * TILE_VECS < vecs && whole_tiles % gridDim.x == blockIdx.x) {
#pragma unroll
    for (int u = 0; u < HIST_UNROLL; ++u) {
      const uint64_t i = whole_tiles * TILE_VECS + threadIdx.x + (uint64_t)u * HIST_BLOCK;
      if (i < vecs) {
        const Vec16<K> x = body[i];
#pragma unroll
        for (int j = 0; j < VEC; ++j) count(x.v[j]);
      }
    }
  }
  __syncthreads();
  // fold the copies; thread t starts at copy t so that a wave spreads over all banks
  for (int bin = threadIdx.x; bin < BINS; bin += HIST_BLOCK) {
    uint32_t c = 0;
#pragma unroll 8
    for (int j = 0; j < COPIES; ++j) c += s_hist[bin * COPIES + ((j + threadIdx.x) % COPIES)];
    if (c) atomicAdd(&hist[bin], c);
  }
}

template <typename K>
static void launch_histogram(int passes, uint32_t blocks, hipStream_t stream, const K* keys,
                             uint64_t n, const KeyCodec<K>& codec, const SortGeometry& geo,
                             uint32_t* hist) {
  const bool whole = codec.plain && geo.begin_bit == 0 && geo.end_bit == passes * RADIX_BITS;
#define TA_HIST_CASE(NP)                                                                       \
  case NP:                                                                                     \
    if (whole)                                                                                 \
      TA_LAUNCH("sort_histogram", stream, (sort_histogram_kernel<K, NP, true>), dim3(blocks),  \
                dim3(HIST_BLOCK), keys, n, codec, geo, hist);                                  \
    else                                                                                       \
      TA_LAUNCH("sort_histogram", stream, (sort_histogram_kernel<K, NP, false>), dim3(blocks), \
                dim3(HIST_BLOCK), keys, n, codec, geo, hist);                                  \
    break;
  switch (passes) {
    TA_HIST_CASE(1) TA_HIST_CASE(2) TA_HIST_CASE(3) TA_HIST_CASE(4)
    TA_HIST_CASE(5) TA_HIST_CASE(6) TA_HIST_CASE(7) TA_HIST_CASE(8)
    default: break;
  }
#undef TA_HIST_CASE
}

// ------------------------------------------------------------------ scan of the histograms
// One workgroup of 256 threads; thread d owns bin d.  hist[p][d] becomes the exclusive
// prefix (the global offset of digit d in pass p).
__global__ __launch_bounds__(RADIX_SIZE) void sort_scan_kernel(uint32_t* __restrict__ hist,
                                                               uint32_t n, SortGeometry geo,
                                                               SortCtl* __restrict__ ctl) {
  __shared__ uint32_t s_wave[RADIX_SIZE / WAVE];
  __shared__ uint32_t s_full;
  const int d = threadIdx.x;
  uint32_t parity = 0;
  for (int p = 0; p < geo.passes; ++p) {
    if (d == 0) s_full = 0;
    __syncthreads();
    const uint32_t c = hist[p * RADIX_SIZE + d];
    if (c == n) s_full = 1;
    const uint32_t incl = wave_inclusive_scan(c, OpPlus{});
    if ((d % WAVE) == WAVE - 1) s_wave[d / WAVE] = incl;
    __syncthreads();
    uint32_t base = 0;
    for (int w = 0; w < d / WAVE; ++w) base += s_wave[w];
    hist[p * RADIX_SIZE + d] = base + incl - c;
    const uint32_t skip = s_full;
    if (d == 0) {
      ctl->skip[p] = skip;
      ctl->src_alt[p] = parity;
    }
    parity ^= (skip ? 0u : 1u);
    __syncthreads();
  }
  if (d == 0) {
    ctl->final_in_alt = parity;
    ctl->gave_up = 0;
  }
}

// ------------------------------------------------------------------ onesweep pass
// f(a, b, c) = a & ~(b ^ c): truth table index = a*4 + b*2 + c.
constexpr int BITOP_AND_XNOR = 0x90;

template <typename K, typename V, bool HAS_VALUES, int BLOCK, int ITEMS>
struct PassShape {
  static constexpr int WAVES = BLOCK / WAVE;
  static constexpr int TILE = BLOCK * ITEMS;
  static constexpr size_t EXCH_ITEM = (HAS_VALUES && sizeof(V) > sizeof(K)) ? sizeof(V) : sizeof(K);
  static constexpr size_t EXCH_BYTES = (size_t)TILE * EXCH_ITEM;
  static constexpr size_t CNT_BYTES = (size_t)WAVES * RADIX_SIZE * sizeof(uint32_t);
  static constexpr size_t UNION_BYTES = EXCH_BYTES > CNT_BYTES ? EXCH_BYTES : CNT_BYTES;
};

// Tile descriptors fetched together per look-back round by each digit thread.
constexpr int LOOKBACK_WINDOW = 4;

// OFF32: every key and value of the call lies within 4 GiB of its array's start, so that
// global addresses are a scalar base plus a 32-bit byte offset (one vector instruction per
// access less than with 64-bit address arithmetic).
template <typename K, typename V, bool HAS_VALUES, int BLOCK, int ITEMS, typename D, bool OFF32>
__global__ __launch_bounds__(BLOCK) void onesweep_pass_kernel(
    K* __restrict__ keys_a, K* __restrict__ keys_b, V* __restrict__ vals_a, V* __restrict__ vals_b,
    uint32_t n, int pass, SortGeometry geo, KeyCodec<K> codec,
    const uint32_t* __restrict__ bin_base,  // [RADIX_SIZE] global digit offsets of this pass
    D* __restrict__ status,                 // [tiles][RADIX_SIZE]
    uint32_t* __restrict__ ticket,          // [TICKET_CLASSES] counters of this pass, TICKET_STRIDE words apart
    const SortCtl* __restrict__ ctl,
    uint32_t* __restrict__ gave_up) {       // &SortCtl::gave_up, the one field the passes write
  using Shape = PassShape<K, V, HAS_VALUES, BLOCK, ITEMS>;
  using Desc = Descriptor<D>;
  constexpr int WAVES = Shape::WAVES;
  constexpr int TILE = Shape::TILE;
  static_assert(BLOCK >= RADIX_SIZE, "one thread per digit is required");

  if (ctl->skip[pass]) return;
  const bool from_alt = ctl->src_alt[pass] != 0;
  const K* __restrict__ keys_in = from_alt ? keys_b : keys_a;
  K* __restrict__ keys_out = from_alt ? keys_a : keys_b;
  const V* __restrict__ vals_in = from_alt ? vals_b : vals_a;
  V* __restrict__ vals_out = from_alt ? vals_a : vals_b;

  __shared__ __attribute__((aligned(16))) unsigned char s_union[Shape::UNION_BYTES];
  __shared__ uint32_t s_scatter_base[RADIX_SIZE];  // global offset - local offset, per digit
  __shared__ uint32_t s_digit_wave[RADIX_SIZE / WAVE];
  __shared__ uint32_t s_tile;
  uint32_t* s_cnt = reinterpret_cast<uint32_t*>(s_union);  // [WAVES][RADIX_SIZE]
  K* s_keys = reinterpret_cast<K*>(s_union);
  V* s_vals = reinterpret_cast<V*>(s_union);

  if (threadIdx.x == 0) {
    const uint32_t k = blockIdx.x % TICKET_CLASSES;
    s_tile = class_tile(k, atomicAdd(ticket + k * TICKET_STRIDE, 1u), gridDim.x);
  }
  for (int i = threadIdx.x; i < WAVES * RADIX_SIZE; i += BLOCK) s_cnt[i] = 0;
  __syncthreads();
  const uint32_t tile = __builtin_amdgcn_readfirstlane(s_tile);
  const uint32_t tile_base = tile * (uint32_t)TILE;
  const uint32_t valid = (n - tile_base < (uint32_t)TILE) ? (n - tile_base) : (uint32_t)TILE;
  const int wave = threadIdx.x / WAVE;
  const int lane = threadIdx.x % WAVE;
  const uint32_t span = (uint32_t)wave * (WAVE * ITEMS) + lane;  // + r*64

  const int shift = geo.begin_bit + pass * RADIX_BITS;
  const int nbits = (geo.end_bit - shift) < RADIX_BITS ? (geo.end_bit - shift) : RADIX_BITS;
  const uint32_t dmask = (1u << nbits) - 1u;
  auto digit_of = [&](K x) -> uint32_t {
    if constexpr (sizeof(K) == 8) return __builtin_amdgcn_ubfe((uint32_t)(x >> shift), 0u, (uint32_t)nbits);
    else return __builtin_amdgcn_ubfe((uint32_t)x, (uint32_t)shift, (uint32_t)nbits);
  };
  // element i of an array, addressed the cheaper way where the offsets allow it
  auto at = [&](auto* base, uint32_t i) -> auto& {
    using T = std::remove_reference_t<decltype(*base)>;
    if constexpr (OFF32) {
      using B = std::conditional_t<std::is_const<T>::value, const char, char>;
      return *reinterpret_cast<T*>(reinterpret_cast<B*>(base) + (uint32_t)(i * (uint32_t)sizeof(T)));
    } else {
      return base[i];
    }
  };

  // Keys travel between the passes in their encoded form: the first pass that runs encodes them as
  // it loads, the last one decodes them as it stores (unsigned ascending keys need no transform).
  bool encodes = false, decodes = false;  // uniform
  if (!codec.plain) {
    encodes = decodes = true;
    for (int p = 0; p < pass; ++p)
      if (!ctl->skip[p]) encodes = false;
    for (int p = pass + 1; p < geo.passes; ++p)
      if (!ctl->skip[p]) decodes = false;
  }

  // ---- load (wave-striped); slots past the end sort last inside the tile
  K e[ITEMS];
  if (valid == (uint32_t)TILE) {
    const K* __restrict__ tile_keys = keys_in + tile_base;  // scalar
#pragma unroll
    for (int r = 0; r < ITEMS; ++r) e[r] = at(tile_keys, span + r * WAVE);
    if (encodes) {
#pragma unroll
      for (int r = 0; r < ITEMS; ++r) e[r] = codec.encode(e[r]);
    }
  } else {
#pragma unroll
    for (int r = 0; r < ITEMS; ++r) {
      const uint32_t pos = span + r * WAVE;
      K x = (K)~(K)0;
      if (pos < valid) {
        x = keys_in[tile_base + pos];
        if (encodes) x = codec.encode(x);
      }
      e[r] = x;
    }
  }

  // The values start their way now, so that they have arrived by the time the keys have left:
  // loaded only after the look-back, their latency was the longest part of what a tile still
  // had to do once its offsets were known.
  V v[HAS_VALUES ? ITEMS : 1];
  if constexpr (HAS_VALUES) {
    if (valid == (uint32_t)TILE) {
      // whole tile: no predicates, so that all loads are in flight together (a predicated
      // load makes the compiler wait for it before issuing the next one)
      const V* __restrict__ tile_vals = vals_in + tile_base;  // scalar
#pragma unroll
      for (int r = 0; r < ITEMS; ++r) v[r] = at(tile_vals, span + r * WAVE);
    } else {
#pragma unroll
      for (int r = 0; r < ITEMS; ++r) {
        const uint32_t pos = span + r * WAVE;
        v[r] = (pos < valid) ? vals_in[tile_base + pos] : V{};
      }
    }
  }

  // ---- rank inside the wave by digit
  // Per digit bit: v_bfe_i32 (lane's bit as 0 / -1), one ballot, and two v_bitop3 folding
  // "same bit as mine" into the 64-bit peer mask.  The wave-private counter is read by every
  // lane and then raised by the size of the peer group; LDS executes a wave's instructions
  // in order, so the next round reads the updated count.
  uint32_t* my_cnt = s_cnt + wave * RADIX_SIZE;
  // ranks are < TILE <= 65536: two per register
  static_assert(TILE <= 65536 && ITEMS % 2 == 0, "rank packing");
  uint32_t rank2[ITEMS / 2];
#pragma unroll
  for (int r = 0; r < ITEMS; ++r) {
    const uint32_t d = digit_of(e[r]);
    const uint32_t old = my_cnt[d];
    uint32_t peers_lo = ~0u, peers_hi = ~0u;
#pragma unroll
    for (int b = 0; b < RADIX_BITS; ++b) {
      int sb;
      // opaque to the optimiser so that the compare below is made on sb itself
      asm volatile("v_bfe_i32 %0, %1, %2, 1" : "=v"(sb) : "v"(d), "n"(b));
      const uint64_t m = __builtin_amdgcn_ballot_w64(sb != 0);
      peers_lo = __builtin_amdgcn_bitop3_b32(peers_lo, (uint32_t)m, (uint32_t)sb, BITOP_AND_XNOR);
      peers_hi = __builtin_amdgcn_bitop3_b32(peers_hi, (uint32_t)(m >> 32), (uint32_t)sb, BITOP_AND_XNOR);
    }
    // the count of peers in lower lanes is accumulated onto the counter's value
    const uint32_t rank = __builtin_amdgcn_mbcnt_hi(peers_hi, __builtin_amdgcn_mbcnt_lo(peers_lo, old));
    // The lowest lane of every group of peers bumps the counter for all of them: one LDS
    // write per distinct digit instead of an atomic per key, which an LDS bank serialises
    // when many lanes hold the same digit (float exponents, skewed keys).
    if (rank == old) my_cnt[d] = old + (uint32_t)__builtin_popcount(peers_lo) + (uint32_t)__builtin_popcount(peers_hi);
    if (r % 2 == 0) rank2[r / 2] = rank;
    else rank2[r / 2] |= rank << 16;
    // pin the packed rank here: otherwise the add is sunk past the barrier and `old` and
    // `below` of every round stay live
    asm volatile("" : "+v"(rank2[r / 2]));
    // keep the scheduler from computing all peer masks first (two live registers per
    // round): rounds are finished in pairs
    if (r % 2 == 1) __builtin_amdgcn_sched_barrier(0);
  }
  __syncthreads();

  // ---- per digit: offsets of the waves, tile count; publish the tile's partial counts
  uint32_t digit_count = 0;
  D* my_status = status + (size_t)tile * RADIX_SIZE;
  if (threadIdx.x < RADIX_SIZE) {
    const int d = threadIdx.x;
    uint32_t sum = 0;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) {
      const uint32_t c = s_cnt[w * RADIX_SIZE + d];
      s_cnt[w * RADIX_SIZE + d] = sum;
      sum += c;
    }
    digit_count = sum;
    // padding slots carry the all-ones key and must not be counted
    if (d == (int)dmask) digit_count -= ((uint32_t)TILE - valid);
    if (tile != 0)
      __hip_atomic_store(my_status + d, (D)(Desc::PARTIAL | digit_count), __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_AGENT);
    // exclusive scan of the (padded) counts over the digits -> local run offsets;
    // the part inside this wave of 64 digits now, the preceding waves after the barrier
    const uint32_t incl = wave_inclusive_scan(sum, OpPlus{});
    if (lane == WAVE - 1) s_digit_wave[wave] = incl;
    s_scatter_base[d] = incl - sum;
  }
  __syncthreads();
  uint32_t local_base = 0;
  if (threadIdx.x < RADIX_SIZE) {
    const int d = threadIdx.x;
    local_base = s_scatter_base[d];
    for (int w = 0; w < wave; ++w) local_base += s_digit_wave[w];
#pragma unroll
    for (int w = 0; w < WAVES; ++w) s_cnt[w * RADIX_SIZE + d] += local_base;
  }
  __syncthreads();

  // ---- final position of every key inside the tile
#pragma unroll
  for (int r = 0; r < ITEMS; ++r) {
    const uint32_t d = digit_of(e[r]);
    rank2[r / 2] += my_cnt[d] << (16 * (r % 2));  // no carry: each half stays < TILE
  }
  __syncthreads();  // all reads of s_cnt done: the exchange buffer may overwrite it

#pragma unroll
  for (int r = 0; r < ITEMS; ++r) s_keys[(rank2[r / 2] >> (16 * (r % 2))) & 0xffffu] = e[r];

  // ---- look-back: global offset of each digit run of this tile
  // Windowed: the descriptors of the LOOKBACK_WINDOW nearest unread predecessors are
  // fetched together (one memory round trip instead of one per tile), then folded nearest
  // first up to the first inclusive one.  A descriptor not yet published stops the fold;
  // the next window starts at that tile.
  if (threadIdx.x < RADIX_SIZE) {
    const int d = threadIdx.x;
    uint32_t excl;
    if (tile == 0) {
      excl = bin_base[d];
    } else {
      uint32_t acc = 0;
      int t = (int)tile - 1;  // tile counts stay below 2^20
      const D* my_col = status + d;
      uint32_t spins = 0;
      for (;;) {
        D s[LOOKBACK_WINDOW];
#pragma unroll
        for (int k = 0; k < LOOKBACK_WINDOW; ++k) {
          const uint32_t tk = (uint32_t)((t - k) > 0 ? (t - k) : 0);  // tile 0 is always inclusive
          s[k] = __hip_atomic_load(my_col + (size_t)tk * RADIX_SIZE, __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
        }
        __builtin_amdgcn_sched_barrier(0);  // all loads are in flight before the first is used
        bool done = false;
        int used = 0;
#pragma unroll
        for (int k = 0; k < LOOKBACK_WINDOW; ++k) {
          const D flag = s[k] & ~Desc::VALUE_MASK;
          const bool take = !done && used == k && flag != 0;
          if (take) {
            acc += (uint32_t)(s[k] & Desc::VALUE_MASK);
            used = k + 1;
            done = flag == Desc::INCLUSIVE;
          }
        }
        if (done) break;
        t -= used;
        if (used < LOOKBACK_WINDOW) {
          __builtin_amdgcn_s_sleep(1);
          ++spins;
          if (spins >= LOOKBACK_SPIN_LIMIT ||
              (spins % 1024u == 0 &&
               __hip_atomic_load(gave_up, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0)) {
            __hip_atomic_store(gave_up, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            break;
          }
        }
      }
      excl = acc;
    }
    __hip_atomic_store(my_status + d, (D)(Desc::INCLUSIVE | (D)(uint32_t)(excl + digit_count)), __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
    // (in bytes of a key where the offsets are 32-bit)
    s_scatter_base[d] = OFF32 ? (excl - local_base) * (uint32_t)sizeof(K) : excl - local_base;
  }
  __syncthreads();

  // ---- keys leave in tile-sorted order: consecutive lanes write consecutive addresses
  // Batched so that the 2*ITEMS LDS reads are independent and in flight together.
  uint32_t gpos[ITEMS];
  {
    K ek[ITEMS];
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) ek[k] = s_keys[(uint32_t)k * BLOCK + threadIdx.x];
    // gpos: the key's place in the output, as a byte offset where those fit 32 bits
    auto key_slot = [&](uint32_t g) -> K& {
      if constexpr (OFF32) return *reinterpret_cast<K*>(reinterpret_cast<char*>(keys_out) + g);
      else return keys_out[g];
    };
#pragma unroll
    for (int k = 0; k < ITEMS; ++k)
      gpos[k] = s_scatter_base[digit_of(ek[k])] +
                (OFF32 ? (uint32_t)(threadIdx.x * sizeof(K)) + (uint32_t)(k * BLOCK * sizeof(K))
                       : (uint32_t)k * BLOCK + threadIdx.x);
    if (decodes) {
#pragma unroll
      for (int k = 0; k < ITEMS; ++k) ek[k] = codec.decode(ek[k]);
    }
    if (valid == (uint32_t)TILE) {
#pragma unroll
      for (int k = 0; k < ITEMS; ++k) key_slot(gpos[k]) = ek[k];
    } else {
#pragma unroll
      for (int k = 0; k < ITEMS; ++k)
        if ((uint32_t)k * BLOCK + threadIdx.x < valid) key_slot(gpos[k]) = ek[k];
    }
  }
  if constexpr (HAS_VALUES) {
    __syncthreads();  // keys have been read out of the exchange buffer
#pragma unroll
    for (int r = 0; r < ITEMS; ++r) s_vals[(rank2[r / 2] >> (16 * (r % 2))) & 0xffffu] = v[r];
    __syncthreads();
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
      const uint32_t q = (uint32_t)k * BLOCK + threadIdx.x;
      if constexpr (OFF32) {
        uint32_t vbyte;
        if constexpr (sizeof(V) >= sizeof(K)) vbyte = gpos[k] * (uint32_t)(sizeof(V) / sizeof(K));
        else vbyte = gpos[k] / (uint32_t)(sizeof(K) / sizeof(V));
        if (q < valid) *reinterpret_cast<V*>(reinterpret_cast<char*>(vals_out) + vbyte) = s_vals[q];
      } else {
        if (q < valid) vals_out[gpos[k]] = s_vals[q];
      }
    }
  }
}

// ------------------------------------------------------------------ copy-back
template <typename K, typename V, bool HAS_VALUES>
__global__ __launch_bounds__(256) void sort_copy_back_kernel(K* __restrict__ keys,
                                                             const K* __restrict__ keys_alt,
                                                             V* __restrict__ vals,
                                                             const V* __restrict__ vals_alt,
                                                             uint64_t n,
                                                             const SortCtl* __restrict__ ctl) {
  if (!ctl->final_in_alt) return;
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    keys[i] = keys_alt[i];
    if constexpr (HAS_VALUES) vals[i] = vals_alt[i];
  }
}

// ------------------------------------------------------------------ host side
template <typename K>
static KeyCodec<K> make_codec(int dtype, int descending) {
  KeyCodec<K> c;
  const bool is_float = dtype == THRUST_AMD_F32 || dtype == THRUST_AMD_F64;
  const bool is_signed = is_float || dtype == THRUST_AMD_I8 || dtype == THRUST_AMD_I16 ||
                         dtype == THRUST_AMD_I32 || dtype == THRUST_AMD_I64;
  c.sign = is_signed ? (K)((K)1 << (sizeof(K) * 8 - 1)) : (K)0;
  c.fmask = is_float ? (K)~(K)0 : (K)0;
  c.dmask = descending ? (K)~(K)0 : (K)0;
  c.plain = (!is_signed && !descending) ? 1u : 0u;
  return c;
}

template <typename K, typename V, bool HAS_VALUES>
struct SortPlan {
  // Large tiles (16K-18K keys of 4 bytes) keep the number of tiles in flight, and with it
  // the length of every look-back, small; two blocks of 1024 threads fill a CU (64 VGPRs,
  // 80 KB of LDS each).  8-byte keys or values halve the tile to fit LDS.
  static constexpr int BLOCK = 1024;
  static constexpr int ITEMS = (sizeof(K) == 8 || (HAS_VALUES && sizeof(V) == 8)) ? 8
                               : (sizeof(K) == 4 && !HAS_VALUES)                 ? 18
                                                                                 : 16;
  static constexpr int TILE = BLOCK * ITEMS;
};

template <typename K, typename V, bool HAS_VALUES>
static int sort_impl(void* temp, size_t* temp_bytes, void* keys, void* values, uint64_t n, int dtype,
                     int descending, int begin_bit, int end_bit, hipStream_t stream) {
  using Plan = SortPlan<K, V, HAS_VALUES>;
  const int key_bits = (int)sizeof(K) * 8;
  if (begin_bit < 0 || end_bit > key_bits || begin_bit > end_bit) return (int)hipErrorInvalidValue;
  if (n > SORT_MAX_N) return (int)hipErrorInvalidValue;
  SortGeometry geo;
  geo.begin_bit = begin_bit;
  geo.end_bit = end_bit;
  geo.passes = (end_bit - begin_bit + RADIX_BITS - 1) / RADIX_BITS;
  const uint64_t tiles = (n + Plan::TILE - 1) / Plan::TILE;

  TempLayout lay;
  const size_t off_ctl = lay.add(sizeof(SortCtl));
  // contiguous zero-initialised region: tickets, histograms, tile descriptors
  const bool wide = n > SORT_MAX_N_NARROW;  // prefixes need more than 30 bits: 64-bit descriptors
  // every key and value within 4 GiB of its array's start: 32-bit byte offsets
  const bool off32 = !wide && n * (uint64_t)((HAS_VALUES && sizeof(V) > sizeof(K)) ? sizeof(V) : sizeof(K)) <= (1ull << 32);
  const size_t zero_words = (size_t)TICKET_WORDS + (size_t)MAX_PASSES * RADIX_SIZE +
                            (size_t)geo.passes * tiles * RADIX_SIZE * (wide ? 2 : 1);
  const size_t off_zero = lay.add(zero_words * sizeof(uint32_t));
  const size_t off_keys = lay.add((size_t)n * sizeof(K));
  const size_t off_vals = lay.add(HAS_VALUES ? (size_t)n * sizeof(V) : 0);
  if (temp == nullptr) {
    *temp_bytes = lay.total;
    return 0;
  }
  if (*temp_bytes < lay.total) return (int)hipErrorInvalidValue;
  if (n <= 1 || geo.passes == 0) return 0;
  if (!keys || (HAS_VALUES && !values)) return (int)hipErrorInvalidValue;

  char* base = static_cast<char*>(temp);
  SortCtl* ctl = reinterpret_cast<SortCtl*>(base + off_ctl);
  uint32_t* zero = reinterpret_cast<uint32_t*>(base + off_zero);
  uint32_t* tickets = zero;
  uint32_t* hist = zero + TICKET_WORDS;
  uint32_t* status = hist + MAX_PASSES * RADIX_SIZE;
  K* keys_a = static_cast<K*>(keys);
  K* keys_b = reinterpret_cast<K*>(base + off_keys);
  V* vals_a = static_cast<V*>(values);
  V* vals_b = reinterpret_cast<V*>(base + off_vals);
  const KeyCodec<K> codec = make_codec<K>(dtype, descending);

  {
    uint64_t blocks = (zero_words + 255) / 256;
    if (blocks > (uint64_t)NUM_CU * 8) blocks = (uint64_t)NUM_CU * 8;
    TA_LAUNCH("sort_init", stream, sort_init_kernel, dim3((uint32_t)blocks), dim3(256), zero, (uint64_t)zero_words);
    TA_CHECK_LAUNCH();
  }
  {
    constexpr uint64_t HT = (uint64_t)HIST_BLOCK * HIST_UNROLL * Vec16<K>::N;
    uint64_t blocks = (n + HT - 1) / HT;
    if (blocks > (uint64_t)NUM_CU) blocks = NUM_CU;
    launch_histogram<K>(geo.passes, (uint32_t)blocks, stream, (const K*)keys_a, n, codec, geo, hist);
    TA_CHECK_LAUNCH();
  }
  TA_LAUNCH("sort_scan", stream, sort_scan_kernel, dim3(1), dim3(RADIX_SIZE), hist, (uint32_t)n, geo, ctl);
  TA_CHECK_LAUNCH();
  for (int p = 0; p < geo.passes; ++p) {
    const size_t status_off = (size_t)p * tiles * RADIX_SIZE;  // in descriptor words
    if (off32) {
      TA_LAUNCH("onesweep_pass", stream, (onesweep_pass_kernel<K, V, HAS_VALUES, Plan::BLOCK, Plan::ITEMS, uint32_t, true>), dim3((uint32_t)tiles), dim3(Plan::BLOCK), keys_a, keys_b, vals_a, vals_b, (uint32_t)n, p, geo, codec, hist + p * RADIX_SIZE, status + status_off, tickets + (size_t)p * TICKET_CLASSES * TICKET_STRIDE, (const SortCtl*)ctl, &ctl->gave_up);
    } else if (wide) {
      TA_LAUNCH("onesweep_pass", stream, (onesweep_pass_kernel<K, V, HAS_VALUES, Plan::BLOCK, Plan::ITEMS, uint64_t, false>), dim3((uint32_t)tiles), dim3(Plan::BLOCK), keys_a, keys_b, vals_a, vals_b, (uint32_t)n, p, geo, codec, hist + p * RADIX_SIZE, reinterpret_cast<uint64_t*>(status) + status_off, tickets + (size_t)p * TICKET_CLASSES * TICKET_STRIDE, (const SortCtl*)ctl, &ctl->gave_up);
    } else {
      TA_LAUNCH("onesweep_pass", stream, (onesweep_pass_kernel<K, V, HAS_VALUES, Plan::BLOCK, Plan::ITEMS, uint32_t, false>), dim3((uint32_t)tiles), dim3(Plan::BLOCK), keys_a, keys_b, vals_a, vals_b, (uint32_t)n, p, geo, codec, hist + p * RADIX_SIZE, status + status_off, tickets + (size_t)p * TICKET_CLASSES * TICKET_STRIDE, (const SortCtl*)ctl, &ctl->gave_up);
    }
    TA_CHECK_LAUNCH();
  }
  {
    uint64_t blocks = (n + 255) / 256;
    if (blocks > (uint64_t)NUM_CU * 8) blocks = (uint64_t)NUM_CU * 8;
    TA_LAUNCH("sort_copy_back", stream, (sort_copy_back_kernel<K, V, HAS_VALUES>), dim3((uint32_t)blocks), dim3(256), keys_a, (const K*)keys_b, vals_a, (const V*)vals_b, n, (const SortCtl*)ctl);
    TA_CHECK_LAUNCH();
  }
  return 0;
}

}  // namespace ta

TA_EXPORT int thrust_amd_sort_keys(void* temp, size_t* temp_bytes, void* keys, uint64_t n,
                                   int key_dtype, int descending, int begin_bit, int end_bit,
                                   void* stream) {
  using namespace ta;
  if (!temp_bytes || !valid_dtype(key_dtype)) return (int)hipErrorInvalidValue;
  return with_item_bytes(thrust_amd_dtype_size(key_dtype), [&](auto kt) {
    using K = typename decltype(kt)::type;
    return sort_impl<K, uint32_t, false>(temp, temp_bytes, keys, nullptr, n, key_dtype, descending,
                                         begin_bit, end_bit, (hipStream_t)stream);
  });
}

TA_EXPORT int thrust_amd_sort_pairs(void* temp, size_t* temp_bytes, void* keys, void* values,
                                    uint64_t n, int key_dtype, size_t value_bytes, int descending,
                                    int begin_bit, int end_bit, void* stream) {
  using namespace ta;
  if (!temp_bytes || !valid_dtype(key_dtype) || !valid_item_bytes(value_bytes))
    return (int)hipErrorInvalidValue;
  return with_item_bytes(thrust_amd_dtype_size(key_dtype), [&](auto kt) {
    using K = typename decltype(kt)::type;
    return with_item_bytes(value_bytes, [&](auto vt) {
      using V = typename decltype(vt)::type;
      return sort_impl<K, V, true>(temp, temp_bytes, keys, values, n, key_dtype, descending,
                                   begin_bit, end_bit, (hipStream_t)stream);
    });
  });
}
