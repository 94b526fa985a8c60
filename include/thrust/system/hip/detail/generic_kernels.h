// reduce and the scans for a user's binary operator or element type: kernels that take
// the operator, the input iterator and the element type as template arguments, so they are
// instantiated in the user's translation unit (hipcc).  The operators of the closed set
// on arithmetic types never come here; they run in the library's tuned kernels.
//
//   reduce  every workgroup folds one contiguous chunk (each lane its own elements, then
//           a tree over the lanes through LDS), a last workgroup folds the chunk results
//           into init.  The operator must be associative and commutative, as the
//           reference requires of reduce.
//   scan    three steps: the fold of every tile (256 lanes, about 64 bytes each); an in-order scan of the tile
//           results (by one workgroup when they are few, else by the same three steps one
//           level up); every tile scanned again with what precedes it.
//           Only associativity is used: operands always meet in input order.
//
// There is no identity for an arbitrary operator, so partial results carry a "holds a
// value" flag where a lane or tile may be empty.  HBM traffic: reduce reads the range
// once; the scans read it twice and write it once, with consecutive lanes on consecutive
// elements (the lanes' own order is made in LDS).
#pragma once
#if !defined(__HIPCC__)
#error "thrust/system/hip/detail/generic_kernels.h is HIP code: compile this translation unit with hipcc"
#endif
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace thrust {
namespace system {
namespace hip {
namespace generic {

constexpr int BLOCK = 256;
constexpr int ITEMS = 8;
constexpr int TILE = BLOCK * ITEMS;

// Fold of the lanes' values in lane order; lanes without a value are skipped.  Returns the
// total in every lane (has_total tells whether any lane held a value).
template <typename T, typename Op>
__device__ __forceinline__ T block_fold(T value, bool has, Op& op, T* s_val, unsigned char* s_has, bool& has_total) {
  const unsigned tid = threadIdx.x;
  s_val[tid] = value;
  s_has[tid] = has ? 1 : 0;
  __syncthreads();
  for (unsigned step = 1; step < BLOCK; step <<= 1) {
    // after this round, lane t (t % (2*step) == 0) holds the fold of lanes [t, t + 2*step)
    if ((tid & (2 * step - 1)) == 0) {
      const bool ha = s_has[tid] != 0, hb = s_has[tid + step] != 0;
      if (ha && hb) s_val[tid] = op(s_val[tid], s_val[tid + step]);
      else if (hb) s_val[tid] = s_val[tid + step];
      s_has[tid] = (ha || hb) ? 1 : 0;
    }
    __syncthreads();
  }
  has_total = s_has[0] != 0;
  const T total = s_val[0];
  __syncthreads();
  return total;
}

// partials[b] = fold of chunk b; every chunk holds at least one element (the host sizes the grid so).
template <typename View, typename T, typename Op>
__global__ __launch_bounds__(BLOCK) void reduce_chunks_kernel(View first, uint64_t n, uint64_t chunk, Op op,
                                                              T* partials) {
  // raw bytes: T may have a constructor, which shared arrays cannot run
  __shared__ __attribute__((aligned(16))) unsigned char s_val_raw[BLOCK * sizeof(T)];
  T* s_val = reinterpret_cast<T*>(s_val_raw);
  __shared__ unsigned char s_has[BLOCK];
  const uint64_t begin = (uint64_t)blockIdx.x * chunk;
  const uint64_t end = (begin + chunk < n) ? begin + chunk : n;
  T acc = T();
  const bool has = begin + threadIdx.x < end;
  if (has) {
    // the lane's first element starts the fold, the rest follow in index order
    acc = (T)first[begin + threadIdx.x];
#pragma unroll 4
    for (uint64_t i = begin + threadIdx.x + BLOCK; i < end; i += BLOCK) acc = op(acc, (T)first[i]);
  }
  bool any;
  const T total = block_fold(acc, has, op, s_val, s_has, any);
  if (threadIdx.x == 0) partials[blockIdx.x] = total;
}

// *result = op(init, partials[0], ..., partials[count - 1])
template <typename T, typename Op>
__global__ __launch_bounds__(BLOCK) void reduce_final_kernel(const T* partials, uint32_t count, T init, Op op,
                                                             T* result) {
  // raw bytes: T may have a constructor, which shared arrays cannot run
  __shared__ __attribute__((aligned(16))) unsigned char s_val_raw[BLOCK * sizeof(T)];
  T* s_val = reinterpret_cast<T*>(s_val_raw);
  __shared__ unsigned char s_has[BLOCK];
  T acc = T();
  bool has = false;
  for (uint32_t i = threadIdx.x; i < count; i += BLOCK) {
    if (has) acc = op(acc, partials[i]);
    else { acc = partials[i]; has = true; }
  }
  bool any;
  const T total = block_fold(acc, has, op, s_val, s_has, any);
  if (threadIdx.x == 0) *result = any ? op(init, total) : init;
}

// The scans' tile: every lane owns ITEMS consecutive elements, about 64 bytes of them.  A tile
// is loaded and stored with consecutive lanes on consecutive elements and turned into the
// lanes' order through LDS; one spare slot after every ITEMS keeps the lanes, which walk
// their own elements, on different banks.
template <typename T>
struct scan_shape {
  static constexpr int WANTED = 64 / (int)sizeof(T);
  static constexpr int ITEMS = WANTED < 1 ? 1 : (WANTED > 16 ? 16 : WANTED);
  static constexpr int TILE = BLOCK * ITEMS;
  // with one element per lane the two orders are the same and nothing is staged
  static constexpr int SLOTS = ITEMS == 1 ? 1 : TILE + BLOCK;
  __host__ __device__ static constexpr unsigned slot(unsigned e) { return e + e / ITEMS; }
};
constexpr int WAVE_LANES = 64;
constexpr int WAVES = BLOCK / WAVE_LANES;

// LDS executes the instructions of one wave in order, so lanes of a wave exchange values
// through it without a barrier; the compiler only has to keep the accesses where they are.
__device__ __forceinline__ void wave_fence() { asm volatile("" ::: "memory"); }

// Inclusive scan of the lanes' values in lane order: Hillis-Steele inside every wave through
// the wave's own part of s_val / s_has, then the totals of the waves before.  Lanes without a
// value take part as "nothing": incl_has tells whether anything precedes or sits in the lane.
// One barrier inside; s_wave / s_wave_has hold WAVES entries.  Returns the inclusive value.
template <typename T, typename Op>
__device__ __forceinline__ T block_inclusive(T value, bool has, Op& op, T* s_val, unsigned char* s_has, T* s_wave,
                                             unsigned char* s_wave_has, bool& incl_has) {
  const unsigned tid = threadIdx.x, lane = tid % WAVE_LANES, wave = tid / WAVE_LANES;
  T v = value;
  bool h = has;
  for (unsigned step = 1; step < WAVE_LANES; step <<= 1) {
    s_val[tid] = v;
    s_has[tid] = h ? 1 : 0;
    wave_fence();
    if (lane >= step && s_has[tid - step]) {
      const T left = s_val[tid - step];
      v = h ? op(left, v) : left;
      h = true;
    }
    wave_fence();
  }
  if (lane == WAVE_LANES - 1) {
    s_wave[wave] = v;
    s_wave_has[wave] = h ? 1 : 0;
  }
  __syncthreads();
  T before = T();
  bool has_before = false;
  for (unsigned w = 0; w < wave; ++w) {
    if (s_wave_has[w]) {
      before = has_before ? op(before, s_wave[w]) : s_wave[w];
      has_before = true;
    }
  }
  if (has_before) {
    v = h ? op(before, v) : before;
    h = true;
  }
  incl_has = h;
  return v;
}

// The tile's elements into s_tile, consecutive lanes on consecutive elements.
template <typename T, typename View>
__device__ __forceinline__ void load_tile(View first, uint64_t tile_base, unsigned valid, T* s_tile) {
  typedef scan_shape<T> S;
  if (S::ITEMS == 1) return;  // every lane reads its one element itself
  T in[S::ITEMS];
#pragma unroll
  for (int q = 0; q < S::ITEMS; ++q) {
    const unsigned e = (unsigned)q * BLOCK + threadIdx.x;
    if (e < valid) in[q] = (T)first[tile_base + e];
  }
#pragma unroll
  for (int q = 0; q < S::ITEMS; ++q) {
    const unsigned e = (unsigned)q * BLOCK + threadIdx.x;
    if (e < valid) s_tile[S::slot(e)] = in[q];
  }
}

#define THRUST_AMD_SCAN_SHARED(T)                                                                      \
  typedef scan_shape<T> S;                                                                             \
  /* raw bytes: T may have a constructor, which shared arrays cannot run */                           \
  __shared__ __attribute__((aligned(16))) unsigned char s_tile_raw[(size_t)S::SLOTS * sizeof(T)];      \
  __shared__ __attribute__((aligned(16))) unsigned char s_val_raw[BLOCK * sizeof(T)];                  \
  __shared__ __attribute__((aligned(16))) unsigned char s_wave_raw[WAVES * sizeof(T)];                 \
  __shared__ unsigned char s_has[BLOCK];                                                               \
  __shared__ unsigned char s_wave_has[WAVES];                                                          \
  T* s_tile = reinterpret_cast<T*>(s_tile_raw);                                                        \
  T* s_val = reinterpret_cast<T*>(s_val_raw);                                                          \
  T* s_wave = reinterpret_cast<T*>(s_wave_raw);

// Step 1 of the scan: tile_total[t] = fold of tile t in input order (every tile holds an element).
template <typename View, typename T, typename Op>
__global__ __launch_bounds__(BLOCK) void scan_tile_totals_kernel(View first, uint64_t n, Op op, T* tile_total) {
  THRUST_AMD_SCAN_SHARED(T)
  const uint64_t tile_base = (uint64_t)blockIdx.x * S::TILE;
  const unsigned valid = (unsigned)((n - tile_base < (uint64_t)S::TILE) ? (n - tile_base) : (uint64_t)S::TILE);
  load_tile<T>(first, tile_base, valid, s_tile);
  __syncthreads();
  T acc = T();
  bool has = false;
#pragma unroll
  for (int i = 0; i < S::ITEMS; ++i) {
    const unsigned e = threadIdx.x * S::ITEMS + i;
    if (e < valid) {
      const T x = S::ITEMS == 1 ? (T)first[tile_base + e] : s_tile[S::slot(e)];
      if (has) acc = op(acc, x);
      else { acc = x; has = true; }
    }
  }
  bool incl_has;
  const T incl = block_inclusive(acc, has, op, s_val, s_has, s_wave, s_wave_has, incl_has);
  if (threadIdx.x == BLOCK - 1) tile_total[blockIdx.x] = incl;  // the last lane's value covers the tile
}

// Step 2: tile_total[t] becomes the fold of tiles 0 .. t (inclusive), in place, by one workgroup:
// every lane owns a contiguous piece of the array.
template <typename T, typename Op>
__global__ __launch_bounds__(BLOCK) void scan_tile_prefix_kernel(T* tile_total, uint32_t tiles, Op op) {
  // raw bytes: T may have a constructor, which shared arrays cannot run
  __shared__ __attribute__((aligned(16))) unsigned char s_val_raw[BLOCK * sizeof(T)];
  __shared__ __attribute__((aligned(16))) unsigned char s_wave_raw[WAVES * sizeof(T)];
  T* s_val = reinterpret_cast<T*>(s_val_raw);
  T* s_wave = reinterpret_cast<T*>(s_wave_raw);
  __shared__ unsigned char s_has[BLOCK];
  __shared__ unsigned char s_wave_has[WAVES];
  const uint32_t per = (tiles + BLOCK - 1) / BLOCK;
  const uint32_t begin = threadIdx.x * per;
  const uint32_t end = (begin + per < tiles) ? begin + per : tiles;
  T acc = T();
  bool has = false;
  for (uint32_t i = begin; i < end; ++i) {
    if (has) acc = op(acc, tile_total[i]);
    else { acc = tile_total[i]; has = true; }
  }
  bool incl_has;
  const T incl = block_inclusive(acc, has, op, s_val, s_has, s_wave, s_wave_has, incl_has);
  // what precedes this lane's piece: the previous lane's inclusive value
  s_val[threadIdx.x] = incl;
  s_has[threadIdx.x] = incl_has ? 1 : 0;
  __syncthreads();
  T carry = T();
  bool has_carry = false;
  if (threadIdx.x > 0 && s_has[threadIdx.x - 1]) {
    carry = s_val[threadIdx.x - 1];
    has_carry = true;
  }
  for (uint32_t i = begin; i < end; ++i) {
    const T x = tile_total[i];
    const T y = has_carry ? op(carry, x) : x;
    tile_total[i] = y;
    carry = y;
    has_carry = true;
  }
}

// Step 3: the tile scanned in input order on top of what precedes it.
//   inclusive:  out[i] = x0 + ... + xi                    (init is not used)
//   exclusive:  out[i] = init + x0 + ... + x(i-1)
// out may be the input itself: a tile is read completely before any of it is written.
// out: a pointer, or any iterator that kernels can take by value (out[i] = value)
template <bool EXCLUSIVE, typename View, typename T, typename U, typename OutView, typename Op>
__global__ __launch_bounds__(BLOCK) void scan_tiles_kernel(View first, OutView out, uint64_t n, Op op, T init,
                                                           const T* tile_prefix) {
  THRUST_AMD_SCAN_SHARED(T)
  const uint64_t tile_base = (uint64_t)blockIdx.x * S::TILE;
  const unsigned valid = (unsigned)((n - tile_base < (uint64_t)S::TILE) ? (n - tile_base) : (uint64_t)S::TILE);
  load_tile<T>(first, tile_base, valid, s_tile);
  __syncthreads();
  const unsigned mine = threadIdx.x * S::ITEMS;
  T x[S::ITEMS];
  T acc = T();
  bool has = false;
#pragma unroll
  for (int i = 0; i < S::ITEMS; ++i) {
    if (mine + i < valid) {
      x[i] = S::ITEMS == 1 ? (T)first[tile_base + mine] : s_tile[S::slot(mine + i)];
      if (has) acc = op(acc, x[i]);
      else { acc = x[i]; has = true; }
    }
  }
  bool incl_has;
  const T incl = block_inclusive(acc, has, op, s_val, s_has, s_wave, s_wave_has, incl_has);
  s_val[threadIdx.x] = incl;  // every wave's scan is behind the barrier inside block_inclusive
  s_has[threadIdx.x] = incl_has ? 1 : 0;
  __syncthreads();
  // carry = everything before this lane's first element: init (exclusive form), the tiles
  // before this one, the lanes before this one
  T carry = T();
  bool has_carry = false;
  if (EXCLUSIVE) {
    carry = init;
    has_carry = true;
  }
  if (blockIdx.x > 0) {
    const T before = tile_prefix[blockIdx.x - 1];
    carry = has_carry ? op(carry, before) : before;
    has_carry = true;
  }
  if (threadIdx.x > 0 && s_has[threadIdx.x - 1]) {
    const T before = s_val[threadIdx.x - 1];
    carry = has_carry ? op(carry, before) : before;
    has_carry = true;
  }
  // results go back to the lane's own slots, then out with consecutive lanes on consecutive elements
#pragma unroll
  for (int i = 0; i < S::ITEMS; ++i) {
    if (mine + i < valid) {
      if (EXCLUSIVE) {
        if (S::ITEMS == 1) out[tile_base + mine] = (U)carry;
        else s_tile[S::slot(mine + i)] = carry;  // has_carry is always true here
        carry = op(carry, x[i]);
      } else {
        carry = has_carry ? op(carry, x[i]) : x[i];
        has_carry = true;
        if (S::ITEMS == 1) out[tile_base + mine] = (U)carry;
        else s_tile[S::slot(mine + i)] = carry;
      }
    }
  }
  if (S::ITEMS == 1) return;
  __syncthreads();
#pragma unroll
  for (int q = 0; q < S::ITEMS; ++q) {
    const unsigned e = (unsigned)q * BLOCK + threadIdx.x;
    if (e < valid) out[tile_base + e] = (U)s_tile[S::slot(e)];
  }
}
#undef THRUST_AMD_SCAN_SHARED

}  // namespace generic
}  // namespace hip
}  // namespace system
}  // namespace thrust
