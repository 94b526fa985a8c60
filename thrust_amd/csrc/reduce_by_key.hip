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
template <typename K, typename V, typename Op>
__global__ __launch_bounds__(RBK_BLOCK, 4) void rbk_kernel(RbkArgs<K, V> a) {
  constexpr int VEC = Vec16<K>::N;
  constexpr int CHUNKS = RBK_ITEMS / VEC >= 1 ? RBK_ITEMS / VEC : 1;
  constexpr int WAVES = RBK_BLOCK / WAVE;
  constexpr uint32_t WAVE_SPAN = WAVE * CHUNKS * VEC;
  constexpr uint32_t TILE = WAVES * WAVE_SPAN;
  using WV = typename SegValue<V>::type;
  using Pair = SegPair<WV>;
  using VV = RbkValueVec<V, VEC>;
  const SegOp<V, Op> sop{Op{}};
  const V vid = Op::template identity<V>();
  const Pair pid{0u, (WV)vid};

  __shared__ uint32_t s_tile;
  __shared__ Pair s_wave_agg[WAVES];
  __shared__ Pair s_prefix;

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

  // ---- head / tail flags per chunk (bit i = element i), lane-local inclusive pairs
  uint32_t head[CHUNKS], tail[CHUNKS];
  Pair lane_excl[CHUNKS];
  Pair carry = pid;
#pragma unroll
  for (int j = 0; j < CHUNKS; ++j) {
    const uint64_t first = tile_base + lane_off + j * (WAVE * VEC);
    K prev = dpp_move<0x138 /* wave_shr:1 */>(k[j].v[VEC - 1], k[j].v[VEC - 1]);
    K next = dpp_move<0x130 /* wave_shl:1 */>(k[j].v[0], k[j].v[0]);
    bool first_of_all = false, last_of_all = false;
    if (lane == 0) {
      if (first == 0) first_of_all = true;
      else if (first < a.n) prev = a.keys[first - 1];
    }
    if (lane == WAVE - 1) {
      if (first + VEC < a.n) next = a.keys[first + VEC];
    }
    uint32_t h = 0, t = 0;
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      const uint64_t pos = first + i;
      const K p = (i == 0) ? prev : k[j].v[i - 1];
      const K nx = (i == VEC - 1) ? next : k[j].v[i + 1];
      const bool in_range = pos < a.n;
      const bool hd = in_range && ((i == 0 && first_of_all) || !(p == k[j].v[i]));
      const bool tl = in_range && (pos + 1 == a.n || !(k[j].v[i] == nx));
      h |= (uint32_t)hd << i;
      t |= (uint32_t)tl << i;
    }
    (void)last_of_all;
    head[j] = h;
    tail[j] = t;
    // fold of the lane's VEC elements
    Pair agg{h & 1u, (WV)v[j].v[0]};
#pragma unroll
    for (int i = 1; i < VEC; ++i) agg = sop(agg, Pair{(h >> i) & 1u, (WV)v[j].v[i]});
    const Pair incl = wave_inclusive_scan(agg, sop, pid);
    lane_excl[j] = sop(carry, dpp_move<0x138>(pid, incl));
    carry = sop(carry, readlane(incl, WAVE - 1));
  }
  if (lane == 0) s_wave_agg[wave] = carry;
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
  const Pair before_wave = sop(s_prefix, wave_prefix);

  // ---- emit first keys at run beginnings, run totals at run ends
#pragma unroll
  for (int j = 0; j < CHUNKS; ++j) {
    Pair run = sop(before_wave, lane_excl[j]);
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      run = sop(run, Pair{(head[j] >> i) & 1u, (WV)v[j].v[i]});
      if ((head[j] >> i) & 1u) a.keys_out[run.heads - 1] = k[j].v[i];
      if ((tail[j] >> i) & 1u) a.values_out[run.heads - 1] = (V)run.value;
    }
  }
}

template <typename K, typename V, typename Op>
static int rbk_run(void* temp, size_t* temp_bytes, const void* keys_in, const void* values_in,
                   void* keys_out, void* values_out, uint64_t* d_num_runs, uint64_t n,
                   hipStream_t stream) {
  constexpr int VEC = Vec16<K>::N;
  constexpr int CHUNKS = RBK_ITEMS / VEC >= 1 ? RBK_ITEMS / VEC : 1;
  constexpr uint64_t TILE = (uint64_t)RBK_BLOCK * CHUNKS * VEC;
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
  TA_LAUNCH("reduce_by_key", stream, (rbk_kernel<K, V, Op>), dim3((uint32_t)tiles), dim3(RBK_BLOCK), a);
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
