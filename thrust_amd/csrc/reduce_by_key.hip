// thrust_amd_reduce_by_key: single-pass segmented reduction.
//
// Every element carries the pair (heads, value): `heads` counts run beginnings, `value`
// is the fold of the values since the last run beginning.  Pairs combine with
//   (h1, v1) (+) (h2, v2) = (h1 + h2, h2 ? v2 : v1 OP v2)
// which is associative, so the same lane -> wave (DPP) -> workgroup (LDS) -> grid
// (decoupled look-back, dynamic tile ticket) scan as everywhere else applies.  With the
// inclusive pair (H, S) at element i: the run's first key goes to keys_out[H-1] at a run
// beginning, and the run total S goes to values_out[H-1] at a run end.
//
// Inside a run the values are folded in a tree order, so floating-point sums agree
// with the reference's strict left fold (the OMP back end's scan is sequential,
// thrust/system/omp/detail/scan.h:21-22) only to rounding.
//
// HBM traffic: n*(key + value) read, runs*(key + value) written, 8*W bytes of tile
// descriptor per tile.  Replaces ReduceByKeyAgent
// (thrust/system/cuda/detail/reduce_by_key.h:197-836).
#include "common.hpp"
#include "dispatch.hpp"
#include "launch.hpp"
#include "segmented.hpp"

namespace ta {

template <typename K, typename V>
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
};

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

// K is the key's comparison class: an unsigned integer type of the key's size (integer
// keys are equal iff their bits are) or float / double (operator==).
//
// Layout: a lane owns ITEMS = 16 or 20 consecutive elements (four or five 16-byte key vectors
// for 4-byte keys), so the flags and the lane's fold are a serial pass over registers and the whole
// tile needs ONE wave scan of pairs per wave.  (Lanes of a wave then read 16-byte pieces
// 64 bytes apart; the four loads of a lane cover its cache lines completely.)
template <typename K, typename V, typename Op>
__global__ __launch_bounds__((RbkItems<K, V>::block), 4) void rbk_kernel(RbkArgs<K, V> a) {
  constexpr int RBK_BLOCK = RbkItems<K, V>::block;
  constexpr int VEC = Vec16<K>::N;
  constexpr int CHUNKS = RbkItems<K, V>::value / VEC >= 1 ? RbkItems<K, V>::value / VEC : 1;
  constexpr int ITEMS = CHUNKS * VEC;
  constexpr int WAVES = RBK_BLOCK / WAVE;
  constexpr uint32_t TILE = RBK_BLOCK * ITEMS;
  using WV = typename SegValue<V>::type;
  using Pair = SegPair<WV>;
  using VV = RbkValueVec<V, VEC>;
  const SegOp<V, Op> sop{Op{}};
  const V vid = Op::template identity<V>();
  const Pair pid{0u, (WV)vid};

  // Outputs of a tile with RBK_SPARSE .. RBK_STAGED runs are gathered in LDS and leave in
  // coalesced stores.  A tile with more runs writes them directly (its run beginnings are
  // dense, so neighbouring lanes write neighbouring addresses anyway), and so does a tile
  // with very few (nothing to coalesce; its waves retire without another barrier).
  constexpr uint32_t RBK_STAGED = 4096;
  constexpr uint32_t RBK_SPARSE = 128;
  __shared__ uint32_t s_tile;
  __shared__ Pair s_wave_agg[WAVES];
  __shared__ Pair s_prefix;
  __shared__ K s_keys_out[RBK_STAGED];
  __shared__ V s_values_out[RBK_STAGED + 1];
  __shared__ uint32_t s_first_is_head, s_last_is_tail;

  if (threadIdx.x == 0) s_tile = atomicAdd(a.ticket, 1u);
  __syncthreads();
  const uint32_t tile = s_tile;
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
  for (int i = 0; i < ITEMS; ++i) differs |= (uint32_t)(!(((i == 0) ? prev : k[i - 1]) == k[i])) << i;
  differs |= (uint32_t)(!(k[ITEMS - 1] == next)) << ITEMS;
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
  const Pair incl = wave_inclusive_scan(agg, sop, pid);
  const Pair lane_excl = dpp_move<0x138>(pid, incl);
  if (lane == WAVE - 1) s_wave_agg[wave] = incl;
  __syncthreads();
  Pair wave_prefix = pid, tile_agg = pid;
#pragma unroll
  for (int w = 0; w < WAVES; ++w) {
    if (w == wave) wave_prefix = tile_agg;
    tile_agg = sop(tile_agg, s_wave_agg[w]);
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
      excl = tile_lookback<Pair>(a.status, tile, sop, pid);
      if (lane == 0) tile_publish<Pair>(my_slot, TS_INCLUSIVE, sop(excl, tile_agg));
    }
    if (lane == 0) {
      s_prefix = excl;
      if (tile_base + valid == a.n) *a.d_num_runs = (uint64_t)excl.heads + tile_agg.heads;
    }
  }
  __syncthreads();

  // ---- emit first keys at run beginnings, run totals at run ends
  const uint32_t runs_before = s_prefix.heads;  // runs begun before this tile
  const uint32_t tile_runs = tile_agg.heads;    // runs begun in this tile
  Pair run = sop(sop(s_prefix, wave_prefix), lane_excl);
  if (tile_runs > RBK_STAGED || tile_runs < RBK_SPARSE) {
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
      run = sop(run, Pair{(head >> i) & 1u, (WV)v[i]});
      if ((head >> i) & 1u) a.keys_out[run.heads - 1] = k[i];
      if ((tail >> i) & 1u) a.values_out[run.heads - 1] = (V)run.value;
    }
    return;
  }
  // Run r (global index) keeps its key in slot r - runs_before and its total in slot
  // r - runs_before + 1: slot 0 of the totals belongs to a run that began in an earlier
  // tile and ends here.
  if (threadIdx.x == 0) s_first_is_head = head & 1u;
  if (valid - 1 >= lane_off && valid - 1 - lane_off < (uint32_t)ITEMS) s_last_is_tail = (tail >> (valid - 1 - lane_off)) & 1u;
#pragma unroll
  for (int i = 0; i < ITEMS; ++i) {
    run = sop(run, Pair{(head >> i) & 1u, (WV)v[i]});
    if ((head >> i) & 1u) s_keys_out[run.heads - 1 - runs_before] = k[i];
    if ((tail >> i) & 1u) s_values_out[run.heads - runs_before] = (V)run.value;
  }
  __syncthreads();
  for (uint32_t j = threadIdx.x; j < tile_runs; j += RBK_BLOCK) a.keys_out[(uint64_t)runs_before + j] = s_keys_out[j];
  // totals present: every run touched by the tile except a last one that goes on
  const uint32_t lo = s_first_is_head ? 1u : 0u;
  const uint32_t hi = s_last_is_tail ? tile_runs + 1u : tile_runs;  // exclusive
  for (uint32_t j = lo + threadIdx.x; j < hi; j += RBK_BLOCK)
    a.values_out[(uint64_t)runs_before + j - 1] = s_values_out[j];
}

template <typename K, typename V, typename Op>
static int rbk_run(void* temp, size_t* temp_bytes, const void* keys_in, const void* values_in,
                   void* keys_out, void* values_out, uint64_t* d_num_runs, uint64_t n,
                   hipStream_t stream) {
  constexpr int VEC = Vec16<K>::N;
  constexpr int CHUNKS = RbkItems<K, V>::value / VEC >= 1 ? RbkItems<K, V>::value / VEC : 1;
  constexpr int BLOCK = RbkItems<K, V>::block;
  constexpr uint64_t TILE = (uint64_t)BLOCK * CHUNKS * VEC;
  using Pair = SegPair<typename SegValue<V>::type>;
  constexpr int W = TileWords<Pair>::W;
  const uint64_t tiles = (n + TILE - 1) / TILE;
  if (tiles > 0xffffffffull || n > 0xffffffffull) return (int)hipErrorInvalidValue;
  TempLayout lay;
  const size_t off_ticket = lay.add(sizeof(uint32_t));
  const size_t off_status = lay.add((size_t)tiles * W * sizeof(uint64_t));
  if (!temp) {
    *temp_bytes = lay.total;
    return 0;
  }
  if (*temp_bytes < lay.total || !d_num_runs) return (int)hipErrorInvalidValue;
  if (n && (!keys_in || !values_in || !keys_out || !values_out)) return (int)hipErrorInvalidValue;
  char* base = static_cast<char*>(temp);
  RbkArgs<K, V> a{};
  a.keys = static_cast<const K*>(keys_in);
  a.values = static_cast<const V*>(values_in);
  a.keys_out = static_cast<K*>(keys_out);
  a.values_out = static_cast<V*>(values_out);
  a.d_num_runs = d_num_runs;
  a.n = n;
  a.ticket = reinterpret_cast<uint32_t*>(base + off_ticket);
  a.status = reinterpret_cast<uint64_t*>(base + off_status);
  a.aligned = is_aligned16(keys_in) &&
              (reinterpret_cast<uintptr_t>(values_in) % alignof(RbkValueVec<V, VEC>)) == 0;
  const uint64_t words = tiles * W;
  const uint64_t init_threads = words ? words : 1;
  TA_LAUNCH("rbk_init", stream, rbk_init_kernel, dim3((uint32_t)((init_threads + 255) / 256)), dim3(256),
            a.status, words, a.ticket, d_num_runs);
  TA_CHECK_LAUNCH();
  if (n == 0) return 0;
  TA_LAUNCH("reduce_by_key", stream, (rbk_kernel<K, V, Op>), dim3((uint32_t)tiles), dim3(BLOCK), a);
  TA_CHECK_LAUNCH();
  return 0;
}

}  // namespace ta

TA_EXPORT int thrust_amd_reduce_by_key(void* temp, size_t* temp_bytes, const void* keys_in,
                                       const void* values_in, void* keys_out, void* values_out,
                                       uint64_t* d_num_runs, uint64_t n, int key_dtype,
                                       int value_dtype, int op, void* stream) {
  using namespace ta;
  if (!temp_bytes || !valid_dtype(key_dtype) || !valid_dtype(value_dtype) || !valid_binop(op))
    return (int)hipErrorInvalidValue;
  auto by_value = [&](auto kt) {
    using K = typename decltype(kt)::type;
    return with_dtype(value_dtype, [&](auto vt) {
      using V = typename decltype(vt)::type;
      return with_binop(op, [&](auto o) {
        return rbk_run<K, V, decltype(o)>(temp, temp_bytes, keys_in, values_in, keys_out, values_out,
                                          d_num_runs, n, (hipStream_t)stream);
      });
    });
  };
  if (key_dtype == THRUST_AMD_F32) return by_value(TypeTag<float>{});
  if (key_dtype == THRUST_AMD_F64) return by_value(TypeTag<double>{});
  return with_item_bytes(thrust_amd_dtype_size(key_dtype), by_value);
}
