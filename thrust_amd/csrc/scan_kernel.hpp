// Single-pass prefix scan with decoupled look-back: the kernel and its launcher, shared by
// the plain scans (scan.hip) and the scans of a transformed input (transform_scan.hip).
// `Pre` is applied to every element as it is loaded; everything after that is the same.
//
// Tile order is a dynamic ticket (one atomic per workgroup), so a tile only ever waits
// for tiles that have already started: correct under any workgroup scheduling order.
// Data layout inside a tile ("wave-striped vectors"): wave w owns a contiguous span of
// 64*CHUNKS 16-byte vectors; its lane l holds vectors l, 64+l, 128+l, ... of that span.
// Every global load/store instruction of a wave therefore covers 1 KiB of consecutive
// addresses, and no LDS transpose is needed: the scan runs as CHUNKS wave scans (DPP)
// chained by the wave total, then one cross-wave step through LDS.
//
// HBM traffic: n*sizeof(T) read + n*sizeof(T) written; tile descriptors add
// 8*W bytes per tile (W = 32-bit words of T).
#pragma once
#include "common.hpp"
#include "dispatch.hpp"
#include "launch.hpp"

namespace ta {

// Tile shapes (threads x 16-byte vectors per lane).  The per-tile cost of the ticket
// (a same-address atomic retires every ~12 ns on MI355X) and of the look-back makes large
// tiles win once there are enough of them to fill 256 CUs; small inputs use small tiles.
struct ScanShapeLarge { static constexpr int BLOCK = 1024, CHUNKS = 12; };
struct ScanShapeSmall { static constexpr int BLOCK = 256, CHUNKS = 4; };
constexpr uint64_t SCAN_LARGE_MIN_BYTES = (uint64_t)32 << 20;

static __global__ void tile_state_init_kernel(uint64_t* __restrict__ words, uint64_t count,
                                       uint32_t* __restrict__ counters, uint32_t num_counters) {
  const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) words[i] = 0;
  if (i < num_counters) counters[i] = 0;
}

// Previous lane's value (lane 0 receives `id`).
template <typename T>
TA_DEVICE T wave_shift_up(T v, T id) {
  return dpp_move<0x138 /* wave_shr:1 */>(id, v);
}

// `finished`, when given, makes the kernel leave its descriptors the way it found them: every tile
// counts itself in once its look-back is over, and the tile that completes the count clears the
// descriptors, the ticket and the counter again.  Storage that is only ever used that way (the
// library's own, all zero when the module is loaded) needs no clearing launch in front of the kernel.
template <typename T, typename Op, typename Pre, bool EXCLUSIVE, bool ALIGNED, typename Shape>
__global__ __launch_bounds__(Shape::BLOCK) void scan_kernel(const T* in, T* out, uint64_t n, T init,
                                                          uint64_t* __restrict__ status,
                                                          uint32_t* __restrict__ ticket,
                                                          uint32_t* __restrict__ finished) {
  constexpr int SCAN_BLOCK = Shape::BLOCK;
  constexpr int SCAN_CHUNKS = Shape::CHUNKS;
  constexpr int VEC = Vec16<T>::N;
  constexpr int WAVES = SCAN_BLOCK / WAVE;
  constexpr uint32_t WAVE_SPAN = WAVE * SCAN_CHUNKS * VEC;  // elements per wave
  constexpr uint32_t TILE = WAVES * WAVE_SPAN;
  constexpr int W = TileWords<T>::W;
  const Op op;
  const Pre pre;
  const T id = Op::template identity<T>();

  __shared__ uint32_t s_tile;
  __shared__ T s_wave_agg[WAVES];
  __shared__ T s_prefix;
  __shared__ uint32_t s_last;

  if (threadIdx.x == 0) {
    s_tile = atomicAdd(ticket, 1u);
    s_last = 0;
  }
  __syncthreads();
  const uint32_t tile = s_tile;
  const uint64_t tile_base = (uint64_t)tile * TILE;
  const uint32_t valid = (uint32_t)((n - tile_base < TILE) ? (n - tile_base) : TILE);
  const int wave = threadIdx.x / WAVE;
  const int lane = threadIdx.x % WAVE;
  const uint32_t lane_off = wave * WAVE_SPAN + lane * VEC;  // + j*64*VEC per chunk

  // ---- load
  Vec16<T> x[SCAN_CHUNKS];
  if (valid == TILE) {
#pragma unroll
    for (int j = 0; j < SCAN_CHUNKS; ++j)
      x[j] = load_vec<ALIGNED>(in + tile_base + lane_off + j * (WAVE * VEC));
#pragma unroll
    for (int j = 0; j < SCAN_CHUNKS; ++j) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) x[j].v[i] = pre(x[j].v[i]);
    }
  } else {
#pragma unroll
    for (int j = 0; j < SCAN_CHUNKS; ++j) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        const uint32_t e = lane_off + j * (WAVE * VEC) + i;
        x[j].v[i] = (e < valid) ? pre(in[tile_base + e]) : id;
      }
    }
  }

  // ---- the tile's aggregate first, and published at once: a later tile's look-back can pass
  // this tile as soon as the sum is known, it does not have to wait for the scan below
  // (plus, minimum and maximum commute, so the lanes may fold their own elements first)
  {
    T lane_total = id;
#pragma unroll
    for (int j = 0; j < SCAN_CHUNKS; ++j) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) lane_total = op(lane_total, x[j].v[i]);
    }
    const T wave_total = wave_reduce(lane_total, op);
    if (lane == 0) s_wave_agg[wave] = wave_total;
  }
  __syncthreads();
  T wave_prefix = id;
  T block_agg = id;
#pragma unroll
  for (int w = 0; w < WAVES; ++w) {
    if (w == wave) wave_prefix = block_agg;
    block_agg = op(block_agg, s_wave_agg[w]);
  }
  uint64_t* my_slot = status + (size_t)tile * W;
  if (threadIdx.x == 0) tile_publish<T>(my_slot, tile == 0 ? TS_INCLUSIVE : TS_PARTIAL, block_agg);

  // ---- wave-local scan in place: every element becomes the fold of the wave's span up to
  // it (inclusive), or up to but excluding it (exclusive); CHUNKS DPP wave scans chained by
  // the wave total.  Nothing but x[] and the carry stays live.
  T carry = id;  // fold of this wave's chunks before chunk j
#pragma unroll
  for (int j = 0; j < SCAN_CHUNKS; ++j) {
    T s = x[j].v[0];
#pragma unroll
    for (int i = 1; i < VEC; ++i) s = op(s, x[j].v[i]);
    const T incl = wave_inclusive_scan(s, op, id);
    T run = op(carry, wave_shift_up(incl, id));
    carry = op(carry, readlane(incl, WAVE - 1));
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      if constexpr (EXCLUSIVE) {
        const T next = op(run, x[j].v[i]);
        x[j].v[i] = run;
        run = next;
      } else {
        run = op(run, x[j].v[i]);
        x[j].v[i] = run;
      }
    }
  }

  // ---- cross-tile prefix
  if (wave == 0) {
    T tile_excl = id;
    if (tile != 0) {
      tile_excl = tile_lookback<T>(status, tile, op, id);
      if (lane == 0) tile_publish<T>(my_slot, TS_INCLUSIVE, op(tile_excl, block_agg));
    }
    if (lane == 0) {
      s_prefix = tile_excl;
      // Counted in only after this tile's last descriptor store has been acknowledged (the wait
      // below; descriptor stores and this counter are agent-scope accesses that bypass the
      // non-coherent caches, so no cache write-back is involved -- a release fence here would
      // write back the L2 with the kernel's output in it, once per tile).  Whoever completes the
      // count knows that no descriptor will be read or written again.
      if (finished != nullptr) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        s_last = __hip_atomic_fetch_add(finished, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == gridDim.x - 1;
      }
    }
  }
  __syncthreads();
  T prefix = s_prefix;
  if constexpr (EXCLUSIVE) prefix = (tile == 0) ? init : op(init, prefix);
  prefix = op(prefix, wave_prefix);

  // ---- apply the prefix of everything before this wave and store
#pragma unroll
  for (int j = 0; j < SCAN_CHUNKS; ++j) {
#pragma unroll
    for (int i = 0; i < VEC; ++i) x[j].v[i] = op(prefix, x[j].v[i]);
  }
  if (valid == TILE) {
#pragma unroll
    for (int j = 0; j < SCAN_CHUNKS; ++j)
      store_vec<ALIGNED>(out + tile_base + lane_off + j * (WAVE * VEC), x[j]);
  } else {
#pragma unroll
    for (int j = 0; j < SCAN_CHUNKS; ++j) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        const uint32_t e = lane_off + j * (WAVE * VEC) + i;
        if (e < valid) out[tile_base + e] = x[j].v[i];
      }
    }
  }
  if (s_last) {
    const uint64_t words = (uint64_t)gridDim.x * W;
    for (uint64_t i = threadIdx.x; i < words; i += SCAN_BLOCK) status[i] = 0;
    if (threadIdx.x == 0) {
      *ticket = 0;
      *finished = 0;
    }
  }
}

template <bool EXCLUSIVE, typename Pre>
struct ScanLaunch {
  // kept_clean: `temp` is storage of the library's own that only this function uses and that was all
  // zero to begin with; the kernel then clears up after itself and no clearing launch precedes it.
  template <typename T, typename Op, typename Shape>
  static int run_shape(void* temp, size_t* temp_bytes, const void* in, void* out, uint64_t n,
                       const void* init, hipStream_t stream, bool kept_clean = false) {
    constexpr int W = TileWords<T>::W;
    constexpr uint64_t TILE = (uint64_t)Shape::BLOCK * Shape::CHUNKS * Vec16<T>::N;
    const uint64_t tiles = (n + TILE - 1) / TILE;
    if (tiles > 0xffffffffull) return (int)hipErrorInvalidValue;
    TempLayout lay;
    const size_t off_ticket = lay.add(2 * sizeof(uint32_t));  // the ticket and the count of finished tiles
    const size_t off_status = lay.add((size_t)tiles * W * sizeof(uint64_t));
    if (temp == nullptr) {
      *temp_bytes = lay.total;
      return 0;
    }
    if (*temp_bytes < lay.total) return (int)hipErrorInvalidValue;
    if (n == 0) return 0;
    if (!in || !out) return (int)hipErrorInvalidValue;
    T init_v = Op::template identity<T>();
    if (EXCLUSIVE) {
      if (!init) return (int)hipErrorInvalidValue;
      __builtin_memcpy(&init_v, init, sizeof(T));
    }
    uint32_t* ticket = reinterpret_cast<uint32_t*>(static_cast<char*>(temp) + off_ticket);
    uint64_t* status = reinterpret_cast<uint64_t*>(static_cast<char*>(temp) + off_status);
    const uint64_t words = tiles * W;
    uint32_t* finished = kept_clean ? ticket + 1 : nullptr;
    if (!kept_clean) {
      TA_LAUNCH("tile_state_init", stream, tile_state_init_kernel, dim3((uint32_t)((words + 255) / 256)), dim3(256), status, words, ticket, 2u);
      TA_CHECK_LAUNCH();
    }
    const T* src = static_cast<const T*>(in);
    T* dst = static_cast<T*>(out);
    if (is_aligned16(in) && is_aligned16(out))
      TA_LAUNCH("scan", stream, (scan_kernel<T, Op, Pre, EXCLUSIVE, true, Shape>), dim3((uint32_t)tiles), dim3(Shape::BLOCK), src, dst, n, init_v, status, ticket, finished);
    else
      TA_LAUNCH("scan", stream, (scan_kernel<T, Op, Pre, EXCLUSIVE, false, Shape>), dim3((uint32_t)tiles), dim3(Shape::BLOCK), src, dst, n, init_v, status, ticket, finished);
    TA_CHECK_LAUNCH();
    return 0;
  }

  template <typename T, typename Op>
  static int run(void* temp, size_t* temp_bytes, const void* in, void* out, uint64_t n,
                 const void* init, hipStream_t stream, bool kept_clean = false) {
    if (n * sizeof(T) >= SCAN_LARGE_MIN_BYTES)
      return run_shape<T, Op, ScanShapeLarge>(temp, temp_bytes, in, out, n, init, stream, kept_clean);
    return run_shape<T, Op, ScanShapeSmall>(temp, temp_bytes, in, out, n, init, stream, kept_clean);
  }
};

}  // namespace ta
