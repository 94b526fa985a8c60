// reduce and the scans for a user's binary operator or element type: kernels that take
// the operator, the input iterator and the element type as template arguments, so they are
// instantiated in the user's translation unit (hipcc).  The operators of the closed set
// on arithmetic types never come here; they run in the library's tuned kernels.
//
//   reduce  every workgroup folds one contiguous chunk (each lane its own elements, then
//           a tree over the lanes through LDS), a last workgroup folds the chunk results
//           into init.  The operator must be associative and commutative, as the
//           reference requires of reduce.
//   scan    three steps: the fold of every 2048-element tile; an in-order scan of the tile
//           results by one workgroup; every tile scanned again with what precedes it.
//           Only associativity is used: operands always meet in input order.
//
// There is no identity for an arbitrary operator, so partial results carry a "holds a
// value" flag where a lane or tile may be empty.  HBM traffic: reduce reads the range
// once; the scans read it twice and write it once.
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

// Inclusive scan of the lanes' values in lane order (Hillis-Steele through LDS).  Lanes
// without a value take part as "nothing": incl_has tells whether anything precedes or sits
// in the lane.  Returns the inclusive value.
template <typename T, typename Op>
__device__ __forceinline__ T block_inclusive(T value, bool has, Op& op, T* s_val, unsigned char* s_has, bool& incl_has) {
  const unsigned tid = threadIdx.x;
  T v = value;
  bool h = has;
  for (unsigned step = 1; step < BLOCK; step <<= 1) {
    s_val[tid] = v;
    s_has[tid] = h ? 1 : 0;
    __syncthreads();
    if (tid >= step && s_has[tid - step]) {
      v = h ? op(s_val[tid - step], v) : s_val[tid - step];
      h = true;
    }
    __syncthreads();
  }
  incl_has = h;
  return v;
}

// Step 1 of the scan: tile_total[t] = fold of tile t in input order (every tile holds an element).
template <typename View, typename T, typename Op>
__global__ __launch_bounds__(BLOCK) void scan_tile_totals_kernel(View first, uint64_t n, Op op, T* tile_total) {
  // raw bytes: T may have a constructor, which shared arrays cannot run
  __shared__ __attribute__((aligned(16))) unsigned char s_val_raw[BLOCK * sizeof(T)];
  T* s_val = reinterpret_cast<T*>(s_val_raw);
  __shared__ unsigned char s_has[BLOCK];
  const uint64_t base = (uint64_t)blockIdx.x * TILE + (uint64_t)threadIdx.x * ITEMS;
  T acc = T();
  bool has = false;
#pragma unroll
  for (int i = 0; i < ITEMS; ++i) {
    if (base + i < n) {
      const T x = (T)first[base + i];
      if (has) acc = op(acc, x);
      else { acc = x; has = true; }
    }
  }
  bool any;
  const T total = block_fold(acc, has, op, s_val, s_has, any);
  if (threadIdx.x == 0) tile_total[blockIdx.x] = total;
}

// Step 2: tile_total[t] becomes the fold of tiles 0 .. t (inclusive), in place, by one workgroup:
// every lane owns a contiguous piece of the array.
template <typename T, typename Op>
__global__ __launch_bounds__(BLOCK) void scan_tile_prefix_kernel(T* tile_total, uint32_t tiles, Op op) {
  // raw bytes: T may have a constructor, which shared arrays cannot run
  __shared__ __attribute__((aligned(16))) unsigned char s_val_raw[BLOCK * sizeof(T)];
  T* s_val = reinterpret_cast<T*>(s_val_raw);
  __shared__ unsigned char s_has[BLOCK];
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
  const T incl = block_inclusive(acc, has, op, s_val, s_has, incl_has);
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
template <bool EXCLUSIVE, typename View, typename T, typename U, typename Op>
__global__ __launch_bounds__(BLOCK) void scan_tiles_kernel(View first, U* out, uint64_t n, Op op, T init,
                                                           const T* tile_prefix) {
  // raw bytes: T may have a constructor, which shared arrays cannot run
  __shared__ __attribute__((aligned(16))) unsigned char s_val_raw[BLOCK * sizeof(T)];
  T* s_val = reinterpret_cast<T*>(s_val_raw);
  __shared__ unsigned char s_has[BLOCK];
  const uint64_t base = (uint64_t)blockIdx.x * TILE + (uint64_t)threadIdx.x * ITEMS;
  T x[ITEMS];
  T acc = T();
  bool has = false;
#pragma unroll
  for (int i = 0; i < ITEMS; ++i) {
    if (base + i < n) {
      x[i] = (T)first[base + i];
      if (has) acc = op(acc, x[i]);
      else { acc = x[i]; has = true; }
    }
  }
  bool incl_has;
  const T incl = block_inclusive(acc, has, op, s_val, s_has, incl_has);
  s_val[threadIdx.x] = incl;
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
#pragma unroll
  for (int i = 0; i < ITEMS; ++i) {
    if (base + i < n) {
      if (EXCLUSIVE) {
        out[base + i] = (U)carry;  // has_carry is always true here
        carry = op(carry, x[i]);
      } else {
        carry = has_carry ? op(carry, x[i]) : x[i];
        has_carry = true;
        out[base + i] = (U)carry;
      }
    }
  }
}

}  // namespace generic
}  // namespace hip
}  // namespace system
}  // namespace thrust
