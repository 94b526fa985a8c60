// Stable comparison sort for the device system: the half of thrust::sort that the radix
// path does not take -- user comparators and key types that are not plain arithmetic
// (thrust/system/cuda/detail/sort.h:53-1322: block sort, merge-path partition and merge
// agents; thrust/system/detail/sequential/stable_merge_sort.inl for the semantics).
//
// The kernels are templates on the key, the value and the comparator, so they are
// instantiated where the comparator's type is known: inside libthrust_amd.so for the
// operator< / operator> orders behind thrust_amd_merge_sort_keys / _pairs, and in a user's
// own translation unit (compiled with hipcc) for everything else.  This header is HIP
// code; it needs nothing but the HIP runtime.
//
//   block sort   a workgroup sorts a tile of 4096 elements: every lane sorts its 16
//                elements with an odd-even transposition network (adjacent swaps only
//                when strictly out of order: stable), then eight merge rounds through
//                LDS double the sorted runs (merge path per lane, serial merge)
//   merge pass   sorted runs are merged pairwise, run length doubling per pass: one
//                thread per 4096-output tile finds the tile's split on the merge path
//                of its pair of runs, a workgroup stages the two pieces in LDS and
//                merges them; keys and values leave through LDS in coalesced stores
//
// A tie takes the element of the earlier run (the one with the smaller index), so the
// sort is stable.  A ragged last tile is padded with copies of the tile's greatest
// element; being equal to it and behind it, they stay at the end and are not written.
// HBM traffic: (1 + passes) * 2 * n * (key + value) bytes, passes = ceil(log2(n / 4096)).
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#ifndef THRUST_AMD_MERGE_SORT_LAUNCH
#define THRUST_AMD_MERGE_SORT_LAUNCH(label, stream, kernel, grid, block, ...) \
  hipLaunchKernelGGL(kernel, grid, block, 0, stream, __VA_ARGS__)
#endif

namespace thrust {
namespace system {
namespace hip {
namespace merge_sort {

constexpr int BLOCK = 256;
constexpr int ITEMS = 16;
constexpr int TILE = BLOCK * ITEMS;
// one spare slot after every ITEMS: lane t's run t*ITEMS.. starts at slot t*(ITEMS+1), so
// lanes that walk their own runs stay on different banks
constexpr int SLOTS = TILE + TILE / ITEMS + 1;
__device__ __forceinline__ uint32_t slot_of(uint32_t e) { return e + e / ITEMS; }

// Number of elements taken from A among the first `diag` merged outputs (ties: A first).
template <typename Idx, typename GetA, typename GetB, typename Comp>
__device__ __forceinline__ Idx merge_path(GetA a, Idx na, GetB b, Idx nb, Idx diag, Comp& comp) {
  Idx lo = diag > nb ? diag - nb : 0;
  Idx hi = diag < na ? diag : na;
  while (lo < hi) {
    const Idx mid = (lo + hi) >> 1;
    if (!comp(b(diag - 1 - mid), a(mid))) lo = mid + 1;
    else hi = mid;
  }
  return lo;
}

template <typename K, typename V, bool HAS_VALUES, typename Comp>
__global__ __launch_bounds__(BLOCK) void block_sort_kernel(const K* keys_in, const V* vals_in, K* keys_out,
                                                           V* vals_out, uint64_t n, Comp comp) {
  __shared__ __attribute__((aligned(16))) unsigned char s_keys_raw[(size_t)SLOTS * sizeof(K)];
  __shared__ __attribute__((aligned(16))) unsigned char s_vals_raw[HAS_VALUES ? (size_t)SLOTS * sizeof(V) : 16];
  K* s_keys = reinterpret_cast<K*>(s_keys_raw);
  V* s_vals = reinterpret_cast<V*>(s_vals_raw);
  const uint32_t tid = threadIdx.x;
  const uint64_t tile_base = (uint64_t)blockIdx.x * TILE;
  const uint32_t valid = (uint32_t)((n - tile_base < (uint64_t)TILE) ? (n - tile_base) : (uint64_t)TILE);
  const uint32_t run0 = tid * ITEMS;

  // ---- coalesced load, then every lane picks up its ITEMS consecutive elements
  K k[ITEMS];
  V v[HAS_VALUES ? ITEMS : 1];
#pragma unroll
  for (int q = 0; q < ITEMS; ++q) {
    const uint32_t e = (uint32_t)q * BLOCK + tid;
    if (e < valid) {
      k[q] = keys_in[tile_base + e];
      if constexpr (HAS_VALUES) v[q] = vals_in[tile_base + e];
    }
  }
#pragma unroll
  for (int q = 0; q < ITEMS; ++q) {
    const uint32_t e = (uint32_t)q * BLOCK + tid;
    if (e < valid) {
      s_keys[slot_of(e)] = k[q];
      if constexpr (HAS_VALUES) s_vals[slot_of(e)] = v[q];
    }
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < ITEMS; ++i) {
    const uint32_t e = run0 + i;
    k[i] = s_keys[slot_of(e < valid ? e : 0u)];  // padding is replaced below
    if constexpr (HAS_VALUES) v[i] = s_vals[slot_of(e < valid ? e : 0u)];
  }
  if (valid < (uint32_t)TILE) {
    // greatest element of the tile: per lane, then a tree over the lanes through LDS
    K m = k[0];
#pragma unroll
    for (int i = 1; i < ITEMS; ++i)
      if (run0 + i < valid && comp(m, k[i])) m = k[i];
    __syncthreads();  // all lanes have read their elements
    s_keys[tid] = m;
    __syncthreads();
    for (uint32_t step = BLOCK / 2; step > 0; step >>= 1) {
      if (tid < step) {
        const K x = s_keys[tid], y = s_keys[tid + step];
        s_keys[tid] = comp(x, y) ? y : x;
      }
      __syncthreads();
    }
    m = s_keys[0];
#pragma unroll
    for (int i = 0; i < ITEMS; ++i)
      if (run0 + i >= valid) k[i] = m;
  }

  // ---- the lane's own elements: odd-even transposition, stable
#pragma unroll
  for (int round = 0; round < ITEMS; ++round) {
#pragma unroll
    for (int i = round & 1; i + 1 < ITEMS; i += 2) {
      if (comp(k[i + 1], k[i])) {
        const K t = k[i];
        k[i] = k[i + 1];
        k[i + 1] = t;
        if constexpr (HAS_VALUES) {
          const V u = v[i];
          v[i] = v[i + 1];
          v[i + 1] = u;
        }
      }
    }
  }

  // ---- merge rounds: sorted runs of `width` elements are merged pairwise
  for (uint32_t width = ITEMS; width < (uint32_t)TILE; width <<= 1) {
    __syncthreads();  // the previous round's reads are done
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
      s_keys[slot_of(run0) + i] = k[i];
      if constexpr (HAS_VALUES) s_vals[slot_of(run0) + i] = v[i];
    }
    __syncthreads();
    const uint32_t start = run0 & ~(2 * width - 1);
    const uint32_t diag = run0 - start;
    const uint32_t b_start = start + width;
    uint32_t i = merge_path<uint32_t>([&](uint32_t x) { return s_keys[slot_of(start + x)]; }, width,
                                      [&](uint32_t x) { return s_keys[slot_of(b_start + x)]; }, width, diag, comp);
    uint32_t j = diag - i;
    // slots just past a run are read but never taken: start + width + width <= TILE
    K ka = s_keys[slot_of(start + i)];
    K kb = s_keys[slot_of(b_start + j)];
#pragma unroll
    for (int o = 0; o < ITEMS; ++o) {
      const bool take_b = (j < width) && (i >= width || comp(kb, ka));
      k[o] = take_b ? kb : ka;
      const uint32_t src = take_b ? b_start + j : start + i;
      if constexpr (HAS_VALUES) v[o] = s_vals[slot_of(src)];
      if (take_b) {
        ++j;
        kb = s_keys[slot_of(b_start + j)];
      } else {
        ++i;
        ka = s_keys[slot_of(start + i)];
      }
    }
  }

  // ---- coalesced write-out of the valid part
  __syncthreads();
#pragma unroll
  for (int i = 0; i < ITEMS; ++i) {
    s_keys[slot_of(run0) + i] = k[i];
    if constexpr (HAS_VALUES) s_vals[slot_of(run0) + i] = v[i];
  }
  __syncthreads();
#pragma unroll
  for (int q = 0; q < ITEMS; ++q) {
    const uint32_t e = (uint32_t)q * BLOCK + tid;
    if (e < valid) {
      keys_out[tile_base + e] = s_keys[slot_of(e)];
      if constexpr (HAS_VALUES) vals_out[tile_base + e] = s_vals[slot_of(e)];
    }
  }
}

// Geometry of the pair of runs that output tile `tile` belongs to.
struct PairOfRuns {
  uint64_t a_begin, na, b_begin, nb;  // A = [a_begin, a_begin + na), B follows it
  uint64_t out0;                      // offset of the tile's first output inside the pair
};
template <bool LONE>
__device__ __forceinline__ PairOfRuns pair_of(uint64_t tile, uint64_t run, uint64_t n) {
  PairOfRuns p;
  const uint64_t d0 = tile * TILE;
  if (LONE) {
    // one pair of runs of any two lengths: A = [0, run), B = [run, n) -- thrust::merge of two ranges
    p.a_begin = 0;
    p.na = run;
    p.b_begin = run;
    p.nb = n - run;
    p.out0 = d0;
    return p;
  }
  p.a_begin = d0 / (2 * run) * (2 * run);
  p.na = (n - p.a_begin < run) ? (n - p.a_begin) : run;
  p.b_begin = p.a_begin + p.na;
  p.nb = (n - p.b_begin < run) ? (n - p.b_begin) : run;
  p.out0 = d0 - p.a_begin;
  return p;
}

// split[t] = how many of the outputs of tile t's pair that precede tile t come from run A.
template <typename K, typename Comp, bool LONE = false>
__global__ __launch_bounds__(256) void merge_partition_kernel(const K* keys, uint64_t n, uint64_t run,
                                                              uint64_t tiles, Comp comp, uint64_t* split) {
  const uint64_t t = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= tiles) return;
  const PairOfRuns p = pair_of<LONE>(t, run, n);
  const K* a = keys + p.a_begin;
  const K* b = keys + p.b_begin;
  // The merge-path search over the whole pair of runs, probing at every step the index of its
  // interval that is a multiple of the largest power of two: as many steps as a bisection at
  // worst, but the first steps of all threads of a pair probe the same few elements, which come
  // from the caches instead of each being a miss of its own.
  const uint64_t diag = p.out0;
  uint64_t lo = diag > p.nb ? diag - p.nb : 0;
  uint64_t hi = diag < p.na ? diag : p.na;
  while (lo < hi) {
    const uint64_t last = hi - 1;
    const uint64_t differ = lo ^ last;
    const uint64_t mid = differ ? (last & ~((1ull << (63 - __builtin_clzll(differ))) - 1ull)) : lo;
    if (!comp(b[diag - 1 - mid], a[mid])) lo = mid + 1;
    else hi = mid;
  }
  split[t] = lo;
}

template <typename K, typename V, bool HAS_VALUES, typename Comp, bool LONE = false>
__global__ __launch_bounds__(BLOCK) void merge_pass_kernel(const K* keys_in, const V* vals_in, K* keys_out,
                                                           V* vals_out, uint64_t n, uint64_t run, uint64_t tiles,
                                                           const uint64_t* split, Comp comp) {
  constexpr size_t ITEM = (HAS_VALUES && sizeof(V) > sizeof(K)) ? sizeof(V) : sizeof(K);
  __shared__ __attribute__((aligned(16))) unsigned char s_raw[(size_t)SLOTS * ITEM];
  K* s_keys = reinterpret_cast<K*>(s_raw);
  V* s_vals = reinterpret_cast<V*>(s_raw);
  const uint32_t tid = threadIdx.x;
  const uint64_t tile = blockIdx.x;
  const PairOfRuns p = pair_of<LONE>(tile, run, n);
  const uint64_t pair_len = p.na + p.nb;
  const uint64_t out1 = (p.out0 + TILE < pair_len) ? p.out0 + TILE : pair_len;
  const uint64_t a0 = split[tile];
  const uint64_t a1 = (out1 == pair_len) ? p.na : split[tile + 1];  // same pair: tile + 1 < tiles
  const uint64_t b0 = p.out0 - a0, b1 = out1 - a1;
  const uint32_t ca = (uint32_t)(a1 - a0), cb = (uint32_t)(b1 - b0);
  const uint32_t count = ca + cb;
  const K* a = keys_in + p.a_begin + a0;
  const K* b = keys_in + p.b_begin + b0;
  const uint64_t out_base = p.a_begin + p.out0;

  // ---- stage the keys: A's piece first, then B's (all loads issued before the first LDS write)
  {
    K in[ITEMS];
#pragma unroll
    for (int q = 0; q < ITEMS; ++q) {
      const uint32_t e = (uint32_t)q * BLOCK + tid;
      if (e < count) in[q] = (e < ca) ? a[e] : b[e - ca];
    }
#pragma unroll
    for (int q = 0; q < ITEMS; ++q) {
      const uint32_t e = (uint32_t)q * BLOCK + tid;
      if (e < count) s_keys[e] = in[q];
    }
  }
  __syncthreads();

  // ---- this lane's start on the path, then a serial merge of ITEMS elements
  const uint32_t run0 = tid * ITEMS;
  const uint32_t diag = run0 < count ? run0 : count;
  uint32_t i = merge_path<uint32_t>([&](uint32_t x) { return s_keys[x]; }, ca,
                                    [&](uint32_t x) { return s_keys[ca + x]; }, cb, diag, comp);
  uint32_t j = ca + (diag - i);  // slot of the next element of B's piece
  K k[ITEMS];
  uint32_t src[ITEMS];
  // a slot at or past `count` is read but never taken (count <= TILE < SLOTS)
  K ka = s_keys[i];
  K kb = s_keys[j];
#pragma unroll
  for (int o = 0; o < ITEMS; ++o) {
    const bool take_b = (j < count) && (i >= ca || comp(kb, ka));
    k[o] = take_b ? kb : ka;
    src[o] = take_b ? j : i;
    const uint32_t next = take_b ? ++j : ++i;
    const K nk = s_keys[next];
    if (take_b) kb = nk;
    else ka = nk;
  }
  __syncthreads();  // all keys have been read from the staging area

  // ---- keys leave through LDS so that consecutive lanes write consecutive addresses
#pragma unroll
  for (int o = 0; o < ITEMS; ++o) s_keys[slot_of(run0) + o] = k[o];
  __syncthreads();
#pragma unroll
  for (int q = 0; q < ITEMS; ++q) {
    const uint32_t e = (uint32_t)q * BLOCK + tid;
    if (e < count) keys_out[out_base + e] = s_keys[slot_of(e)];
  }

  if constexpr (HAS_VALUES) {
    const V* va = vals_in + p.a_begin + a0;
    const V* vb = vals_in + p.b_begin + b0;
    __syncthreads();  // the key write-out has read the exchange buffer
    {
      V in[ITEMS];
#pragma unroll
      for (int q = 0; q < ITEMS; ++q) {
        const uint32_t e = (uint32_t)q * BLOCK + tid;
        if (e < count) in[q] = (e < ca) ? va[e] : vb[e - ca];
      }
#pragma unroll
      for (int q = 0; q < ITEMS; ++q) {
        const uint32_t e = (uint32_t)q * BLOCK + tid;
        if (e < count) s_vals[e] = in[q];
      }
    }
    __syncthreads();
    V v[ITEMS];
#pragma unroll
    for (int o = 0; o < ITEMS; ++o) v[o] = s_vals[src[o] < count ? src[o] : 0u];
    __syncthreads();
#pragma unroll
    for (int o = 0; o < ITEMS; ++o) s_vals[slot_of(run0) + o] = v[o];
    __syncthreads();
#pragma unroll
    for (int q = 0; q < ITEMS; ++q) {
      const uint32_t e = (uint32_t)q * BLOCK + tid;
      if (e < count) vals_out[out_base + e] = s_vals[slot_of(e)];
    }
  }
}

struct Layout {
  size_t off_keys, off_vals, off_split, total;
  uint64_t tiles;
};
inline size_t align256(size_t x) { return (x + 255) / 256 * 256; }
template <typename K, typename V, bool HAS_VALUES>
inline Layout layout(uint64_t n) {
  Layout l;
  l.tiles = (n + TILE - 1) / TILE;
  l.off_keys = 0;
  l.off_vals = align256((size_t)n * sizeof(K));
  l.off_split = l.off_vals + (HAS_VALUES ? align256((size_t)n * sizeof(V)) : 0);
  l.total = l.off_split + align256((size_t)(l.tiles + 1) * sizeof(uint64_t));
  if (l.total == 0) l.total = 256;
  return l;
}

// Sorts keys[0, n) (and values with them) in place.  temp == nullptr: size query.
// Returns a hipError_t as int; everything is enqueued on `stream`, nothing blocks.
template <typename K, typename V, bool HAS_VALUES, typename Comp>
int sort(void* temp, size_t* temp_bytes, K* keys, V* vals, uint64_t n, Comp comp, hipStream_t stream) {
  static_assert(sizeof(K) + (HAS_VALUES ? sizeof(V) : 0) <= 32,
                "comparison sort on the device system: key and value together may take 32 bytes");
  if (!temp_bytes) return (int)hipErrorInvalidValue;
  const Layout lay = layout<K, V, HAS_VALUES>(n);
  if (!temp) {
    *temp_bytes = lay.total;
    return 0;
  }
  if (*temp_bytes < lay.total || lay.tiles > 0x7fffffffull) return (int)hipErrorInvalidValue;
  if (n < 2) return 0;
  if (!keys || (HAS_VALUES && !vals)) return (int)hipErrorInvalidValue;
  char* base = static_cast<char*>(temp);
  K* key_buf[2] = {keys, reinterpret_cast<K*>(base + lay.off_keys)};
  V* val_buf[2] = {vals, reinterpret_cast<V*>(base + lay.off_vals)};
  uint64_t* split = reinterpret_cast<uint64_t*>(base + lay.off_split);
  int passes = 0;
  while (((uint64_t)1 << passes) < lay.tiles) ++passes;
  int cur = passes & 1;  // the block sort writes where an even number of passes ends in `keys`
  THRUST_AMD_MERGE_SORT_LAUNCH("merge_sort_block", stream, (block_sort_kernel<K, V, HAS_VALUES, Comp>),
                               dim3((uint32_t)lay.tiles), dim3(BLOCK), (const K*)keys, (const V*)vals, key_buf[cur],
                               val_buf[cur], n, comp);
  hipError_t err = hipPeekAtLastError();
  if (err != hipSuccess) return (int)err;
  uint64_t run = TILE;
  for (int p = 0; p < passes; ++p) {
    THRUST_AMD_MERGE_SORT_LAUNCH("merge_sort_partition", stream, (merge_partition_kernel<K, Comp>),
                                 dim3((uint32_t)((lay.tiles + 255) / 256)), dim3(256), (const K*)key_buf[cur], n, run,
                                 lay.tiles, comp, split);
    err = hipPeekAtLastError();
    if (err != hipSuccess) return (int)err;
    THRUST_AMD_MERGE_SORT_LAUNCH("merge_sort_pass", stream, (merge_pass_kernel<K, V, HAS_VALUES, Comp>),
                                 dim3((uint32_t)lay.tiles), dim3(BLOCK), (const K*)key_buf[cur],
                                 (const V*)val_buf[cur], key_buf[cur ^ 1], val_buf[cur ^ 1], n, run, lay.tiles,
                                 (const uint64_t*)split, comp);
    err = hipPeekAtLastError();
    if (err != hipSuccess) return (int)err;
    cur ^= 1;
    run *= 2;
  }
  return 0;
}

// Merges the sorted ranges both[0, na) and both[na, n) into out (and their values with them);
// ties take the first range first.  split: (tiles + 1) 64-bit words of scratch.
template <typename K, typename V, bool HAS_VALUES, typename Comp>
int merge_two(const K* both, const V* both_values, uint64_t na, uint64_t n, K* out, V* out_values, uint64_t* split,
              Comp comp, hipStream_t stream) {
  if (n == 0) return 0;
  const uint64_t tiles = (n + TILE - 1) / TILE;
  if (tiles > 0x7fffffffull) return (int)hipErrorInvalidValue;
  THRUST_AMD_MERGE_SORT_LAUNCH("merge_sort_partition", stream, (merge_partition_kernel<K, Comp, true>),
                               dim3((uint32_t)((tiles + 255) / 256)), dim3(256), both, n, na, tiles, comp, split);
  hipError_t err = hipPeekAtLastError();
  if (err != hipSuccess) return (int)err;
  THRUST_AMD_MERGE_SORT_LAUNCH("merge_sort_pass", stream, (merge_pass_kernel<K, V, HAS_VALUES, Comp, true>),
                               dim3((uint32_t)tiles), dim3(BLOCK), both, both_values, out, out_values, n, na, tiles,
                               (const uint64_t*)split, comp);
  return (int)hipPeekAtLastError();
}

}  // namespace merge_sort
}  // namespace hip
}  // namespace system
}  // namespace thrust
