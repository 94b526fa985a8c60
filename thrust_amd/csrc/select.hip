// Stream compaction family: thrust_amd_copy_if, thrust_amd_partition_copy,
// thrust_amd_stable_partition, thrust_amd_unique, thrust_amd_unique_by_key.
//
// One single-pass kernel serves all of them.  Every element gets a 0/1 flag
//   PRED   tested[i] CMP threshold                     (copy_if / partition on the data itself)
//   HEAD   i == 0 || tested[i-1] != tested[i]          (unique, unique_by_key)
//   BYTE   tested[i] != 0, tested = uint8 flag array   (stencil forms, after a flagging pass)
// and the exclusive prefix sum of the flags -- inside the lane, then across the wave with
// DPP, across the waves through LDS, across tiles by decoupled look-back with a dynamic
// tile ticket -- is the output position of each selected element; a rejected element goes
// to (its index - selected before it) of the second output when there is one.  Elements
// are written straight from registers: the selected elements of a wave's 1 KiB load are
// contiguous in the output, so the partial-line stores of a wave meet in L2.
//
// Outputs may alias inputs where the header says so: a tile learns its output offset
// only after every earlier tile has published its count, and a tile publishes only after
// all of its own loads have returned (explicit vmcnt(0) wait before the first barrier).
//
// HBM traffic: n*(tested + payload) read, selected (+ rejected) elements written,
// 16 bytes of tile descriptor per tile.  Replaces the CopyIfAgent / PartitionAgent /
// UniqueAgent / UniqueByKeyAgent kernels of the reference
// (thrust/system/cuda/detail/copy_if.h:365-478, partition.h:221-293, unique.h:316-445,
// unique_by_key.h:348-510).
#include "common.hpp"
#include "dispatch.hpp"
#include "launch.hpp"

namespace ta {

enum SelectFlagMode { FLAG_PRED = 0, FLAG_HEAD = 1, FLAG_BYTE = 2 };

constexpr int SELECT_BLOCK = 1024;
constexpr int SELECT_ITEMS = 16;  // elements per lane

template <typename T, typename U>
struct SelectArgs {
  const T* tested;      // array the flags come from
  const U* payload;     // second stream compacted with the same flags (or nullptr)
  T* tested_true;       // selected tested elements (nullptr: not emitted)
  T* tested_false;      // rejected tested elements (nullptr: not emitted)
  U* payload_true;
  U* payload_false;
  uint64_t* d_num_true;
  uint64_t n;
  int cmp;
  T threshold;
  uint64_t* status;
  uint32_t* ticket;
  uint32_t aligned;     // tested (and payload) pointers allow whole-vector loads
};

// VEC elements of U that belong to one 16-byte vector of T.
template <typename U, int VEC>
struct alignas((VEC * sizeof(U)) >= 16 ? 16 : VEC * sizeof(U)) PayloadVec {
  U v[VEC];
};

__global__ __launch_bounds__(256) void select_init_kernel(uint64_t* __restrict__ words,
                                                          uint64_t count,
                                                          uint32_t* __restrict__ ticket,
                                                          uint64_t* __restrict__ d_num) {
  const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) words[i] = 0;
  if (i == 0) {
    *ticket = 0;
    *d_num = 0;
  }
}

template <typename T, typename U, int MODE, bool HAS_PAYLOAD>
__global__ __launch_bounds__(SELECT_BLOCK, 4) void select_kernel(SelectArgs<T, U> a) {
  constexpr int VEC = Vec16<T>::N;
  constexpr int CHUNKS = SELECT_ITEMS / VEC >= 1 ? SELECT_ITEMS / VEC : 1;
  constexpr int WAVES = SELECT_BLOCK / WAVE;
  constexpr uint32_t WAVE_SPAN = WAVE * CHUNKS * VEC;
  constexpr uint32_t TILE = WAVES * WAVE_SPAN;
  using PV = PayloadVec<U, VEC>;

  __shared__ uint32_t s_tile;
  __shared__ uint32_t s_wave_cnt[WAVES];
  __shared__ uint64_t s_prefix;

  if (threadIdx.x == 0) s_tile = atomicAdd(a.ticket, 1u);
  __syncthreads();
  const uint32_t tile = s_tile;
  const uint64_t tile_base = (uint64_t)tile * TILE;
  const uint32_t valid = (uint32_t)((a.n - tile_base < TILE) ? (a.n - tile_base) : TILE);
  const int wave = threadIdx.x / WAVE;
  const int lane = threadIdx.x % WAVE;
  const uint32_t lane_off = wave * WAVE_SPAN + lane * VEC;  // + j*64*VEC
  const bool full = valid == TILE;

  // ---- load
  Vec16<T> x[CHUNKS];
  PV y[HAS_PAYLOAD ? CHUNKS : 1];
  if (full && a.aligned) {
#pragma unroll
    for (int j = 0; j < CHUNKS; ++j) {
      const uint64_t off = tile_base + lane_off + j * (WAVE * VEC);
      x[j] = *reinterpret_cast<const Vec16<T>*>(a.tested + off);
      if constexpr (HAS_PAYLOAD) y[j] = *reinterpret_cast<const PV*>(a.payload + off);
    }
  } else {
#pragma unroll
    for (int j = 0; j < CHUNKS; ++j) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        const uint32_t e = lane_off + j * (WAVE * VEC) + i;
        x[j].v[i] = (e < valid) ? a.tested[tile_base + e] : T{};
        if constexpr (HAS_PAYLOAD) y[j].v[i] = (e < valid) ? a.payload[tile_base + e] : U{};
      }
    }
  }

  // ---- flags (bit i of fl[j] = element i of chunk j is selected)
  uint32_t fl[CHUNKS];
  if constexpr (MODE == FLAG_HEAD) {
#pragma unroll
    for (int j = 0; j < CHUNKS; ++j) {
      // predecessor of the lane's first element: last element of the previous lane, or,
      // for lane 0, the element just before the wave's chunk in memory
      T prev = dpp_move<0x138 /* wave_shr:1 */>(x[j].v[VEC - 1], x[j].v[VEC - 1]);
      const uint64_t first = tile_base + lane_off + j * (WAVE * VEC);
      bool head0 = false;
      if (lane == 0) {
        if (first == 0) head0 = true;
        else if (first < a.n) prev = a.tested[first - 1];
      }
      uint32_t f = 0;
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        const T p = (i == 0) ? prev : x[j].v[i - 1];
        bool h = !(p == x[j].v[i]);
        if (i == 0) h = h || head0;
        f |= (uint32_t)h << i;
      }
      fl[j] = f;
    }
  } else {
#pragma unroll
    for (int j = 0; j < CHUNKS; ++j) {
      uint32_t f = 0;
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        const bool h = (MODE == FLAG_BYTE) ? (x[j].v[i] != (T)0) : apply_cmp(a.cmp, x[j].v[i], a.threshold);
        f |= (uint32_t)h << i;
      }
      fl[j] = f;
    }
  }
  if (!full) {
#pragma unroll
    for (int j = 0; j < CHUNKS; ++j) {
      const uint32_t e0 = lane_off + j * (WAVE * VEC);
      const uint32_t live = (e0 >= valid) ? 0u : ((valid - e0 >= (uint32_t)VEC) ? ((1u << VEC) - 1u) : ((1u << (valid - e0)) - 1u));
      fl[j] &= live;
    }
  }

  // ---- ranks: lane -> wave (DPP scans chained over the chunks) -> workgroup
  uint32_t lane_excl[CHUNKS];
  uint32_t carry = 0;
#pragma unroll
  for (int j = 0; j < CHUNKS; ++j) {
    const uint32_t c = __builtin_popcount(fl[j]);
    const uint32_t incl = wave_inclusive_scan(c, OpPlus{});
    lane_excl[j] = carry + dpp_move<0x138>(0u, incl);
    carry += readlane(incl, WAVE - 1);
  }
  if (lane == 0) s_wave_cnt[wave] = carry;
  // every load of this wave has returned before the tile's count can become visible:
  // in-place callers rely on it (see the file comment)
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  uint32_t wave_prefix = 0, tile_cnt = 0;
#pragma unroll
  for (int w = 0; w < WAVES; ++w) {
    if (w == wave) wave_prefix = tile_cnt;
    tile_cnt += s_wave_cnt[w];
  }

  // ---- selected elements before this tile
  constexpr int W = TileWords<uint64_t>::W;
  uint64_t* my_slot = a.status + (size_t)tile * W;
  if (wave == 0) {
    uint64_t excl = 0;
    if (tile == 0) {
      if (lane == 0) tile_publish<uint64_t>(my_slot, TS_INCLUSIVE, (uint64_t)tile_cnt);
    } else {
      if (lane == 0) tile_publish<uint64_t>(my_slot, TS_PARTIAL, (uint64_t)tile_cnt);
      excl = tile_lookback<uint64_t>(a.status, tile, OpPlus{}, (uint64_t)0);
      if (lane == 0) tile_publish<uint64_t>(my_slot, TS_INCLUSIVE, excl + tile_cnt);
    }
    if (lane == 0) {
      s_prefix = excl;
      if (tile_base + valid == a.n) *a.d_num_true = excl + tile_cnt;
    }
  }
  __syncthreads();
  const uint64_t true_base = s_prefix + wave_prefix;  // + rank inside the wave
  // a rejected element at tile offset e with r selected elements before it in the tile
  // lands at (tile_base - s_prefix) + e - r of the second output
  const uint64_t false_base = tile_base - s_prefix;
  const bool want_false = (a.tested_false != nullptr) || (HAS_PAYLOAD && a.payload_false != nullptr);

  // ---- scatter straight from registers
#pragma unroll
  for (int j = 0; j < CHUNKS; ++j) {
    uint32_t r = lane_excl[j];
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      const bool sel = (fl[j] >> i) & 1u;
      if (sel) {
        const uint64_t pos = true_base + r;
        if (a.tested_true) a.tested_true[pos] = x[j].v[i];
        if constexpr (HAS_PAYLOAD) a.payload_true[pos] = y[j].v[i];
        ++r;
      } else if (want_false) {
        const uint32_t e = lane_off + j * (WAVE * VEC) + i;
        if (e < valid) {
          const uint64_t pos = false_base + e - (wave_prefix + r);
          if (a.tested_false) a.tested_false[pos] = x[j].v[i];
          if constexpr (HAS_PAYLOAD)
            if (a.payload_false) a.payload_false[pos] = y[j].v[i];
        }
      }
    }
  }
}

// Stencil forms: flags[i] = stencil[i] CMP threshold as one byte each.
template <typename T>
__global__ __launch_bounds__(256) void select_flag_kernel(const T* __restrict__ stencil, uint64_t n,
                                                          int cmp, T threshold,
                                                          uint8_t* __restrict__ flags) {
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
    flags[i] = apply_cmp(cmp, stencil[i], threshold) ? 1 : 0;
}

// Second step of the in-place partition: the rejected elements, parked in temp storage
// in order, move behind the selected ones.
template <typename U>
__global__ __launch_bounds__(256) void partition_tail_kernel(U* __restrict__ data,
                                                             const U* __restrict__ parked,
                                                             uint64_t n,
                                                             const uint64_t* __restrict__ d_num_true) {
  const uint64_t t = *d_num_true;
  const uint64_t f = n - t;
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < f; i += stride)
    data[t + i] = parked[i];
}

struct SelectTemp {
  size_t off_ticket, off_status, off_extra, total;
  uint64_t tiles;
};

template <typename T>
static SelectTemp select_layout(uint64_t n, size_t extra_bytes) {
  constexpr int VEC = Vec16<T>::N;
  constexpr int CHUNKS = SELECT_ITEMS / VEC >= 1 ? SELECT_ITEMS / VEC : 1;
  constexpr uint64_t TILE = (uint64_t)SELECT_BLOCK * CHUNKS * VEC;
  SelectTemp t;
  t.tiles = (n + TILE - 1) / TILE;
  TempLayout lay;
  t.off_ticket = lay.add(sizeof(uint32_t));
  t.off_status = lay.add((size_t)t.tiles * TileWords<uint64_t>::W * sizeof(uint64_t));
  t.off_extra = lay.add(extra_bytes);
  t.total = lay.total;
  return t;
}

template <typename T, typename U, int MODE, bool HAS_PAYLOAD>
static int select_launch(char* temp, const SelectTemp& lay, SelectArgs<T, U> a, hipStream_t stream) {
  if (lay.tiles > 0xffffffffull) return (int)hipErrorInvalidValue;
  a.ticket = reinterpret_cast<uint32_t*>(temp + lay.off_ticket);
  a.status = reinterpret_cast<uint64_t*>(temp + lay.off_status);
  constexpr size_t PAY_ALIGN = alignof(PayloadVec<U, Vec16<T>::N>);
  a.aligned = is_aligned16(a.tested) &&
              (!HAS_PAYLOAD || (reinterpret_cast<uintptr_t>(a.payload) % PAY_ALIGN) == 0);
  const uint64_t words = lay.tiles * TileWords<uint64_t>::W;
  const uint64_t init_threads = words ? words : 1;
  TA_LAUNCH("select_init", stream, select_init_kernel, dim3((uint32_t)((init_threads + 255) / 256)),
            dim3(256), a.status, words, a.ticket, a.d_num_true);
  TA_CHECK_LAUNCH();
  if (a.n == 0) return 0;
  TA_LAUNCH("select", stream, (select_kernel<T, U, MODE, HAS_PAYLOAD>), dim3((uint32_t)lay.tiles),
            dim3(SELECT_BLOCK), a);
  TA_CHECK_LAUNCH();
  return 0;
}

static uint32_t stride_grid(uint64_t n) {
  uint64_t blocks = (n + 255) / 256;
  const uint64_t cap = (uint64_t)NUM_CU * 8;
  if (blocks < 1) blocks = 1;
  return (uint32_t)(blocks < cap ? blocks : cap);
}

// Shared body of copy_if / partition_copy / stable_partition.
//   in_place: out_true == in, rejected elements are parked in temp and moved back.
static int select_by_predicate(void* temp, size_t* temp_bytes, const void* in, const void* stencil,
                               void* out_true, void* out_false, uint64_t* d_num, uint64_t n,
                               size_t item_bytes, int stencil_dtype, int cmp, const void* threshold,
                               bool in_place, hipStream_t stream) {
  if (!temp_bytes || !valid_item_bytes(item_bytes) || !valid_dtype(stencil_dtype) || !valid_cmp(cmp))
    return (int)hipErrorInvalidValue;
  const size_t tested_bytes = thrust_amd_dtype_size(stencil_dtype);
  if (!stencil && tested_bytes != item_bytes) return (int)hipErrorInvalidValue;
  if (cmp != THRUST_AMD_NONZERO && !threshold && temp) return (int)hipErrorInvalidValue;
  const size_t park_bytes = in_place ? (size_t)n * item_bytes : 0;

  if (!stencil) {
    return with_dtype(stencil_dtype, [&](auto tt) {
      using T = typename decltype(tt)::type;
      const SelectTemp lay = select_layout<T>(n, park_bytes);
      if (!temp) {
        *temp_bytes = lay.total;
        return 0;
      }
      if (*temp_bytes < lay.total || !d_num || (n && (!in || !out_true))) return (int)hipErrorInvalidValue;
      char* base = static_cast<char*>(temp);
      SelectArgs<T, uint32_t> a{};
      a.tested = static_cast<const T*>(in);
      a.tested_true = static_cast<T*>(out_true);
      a.tested_false = in_place ? reinterpret_cast<T*>(base + lay.off_extra) : static_cast<T*>(out_false);
      a.d_num_true = d_num;
      a.n = n;
      a.cmp = cmp;
      if (threshold) __builtin_memcpy(&a.threshold, threshold, sizeof(T));
      int rc = select_launch<T, uint32_t, FLAG_PRED, false>(base, lay, a, stream);
      if (rc || !in_place || n == 0) return rc;
      TA_LAUNCH("partition_tail", stream, (partition_tail_kernel<T>), dim3(stride_grid(n)), dim3(256),
                static_cast<T*>(out_true), (const T*)(base + lay.off_extra), n, (const uint64_t*)d_num);
      TA_CHECK_LAUNCH();
      return 0;
    });
  }
  // stencil form: byte flags first, then compaction of the items under those flags
  return with_item_bytes(item_bytes, [&](auto ut) {
    using U = typename decltype(ut)::type;
    const size_t flag_bytes = align_up((size_t)n, 256);
    const SelectTemp lay = select_layout<uint8_t>(n, flag_bytes + park_bytes);
    if (!temp) {
      *temp_bytes = lay.total;
      return 0;
    }
    if (*temp_bytes < lay.total || !d_num || (n && (!in || !out_true))) return (int)hipErrorInvalidValue;
    char* base = static_cast<char*>(temp);
    uint8_t* flags = reinterpret_cast<uint8_t*>(base + lay.off_extra);
    U* parked = reinterpret_cast<U*>(base + lay.off_extra + flag_bytes);
    if (n) {
      int rc = with_dtype(stencil_dtype, [&](auto tt) {
        using T = typename decltype(tt)::type;
        T thr{};
        if (threshold) __builtin_memcpy(&thr, threshold, sizeof(T));
        TA_LAUNCH("select_flag", stream, (select_flag_kernel<T>), dim3(stride_grid(n)), dim3(256),
                  static_cast<const T*>(stencil), n, cmp, thr, flags);
        TA_CHECK_LAUNCH();
        return 0;
      });
      if (rc) return rc;
    }
    SelectArgs<uint8_t, U> a{};
    a.tested = flags;
    a.payload = static_cast<const U*>(in);
    a.payload_true = static_cast<U*>(out_true);
    a.payload_false = in_place ? parked : static_cast<U*>(out_false);
    a.d_num_true = d_num;
    a.n = n;
    int rc = select_launch<uint8_t, U, FLAG_BYTE, true>(base, lay, a, stream);
    if (rc || !in_place || n == 0) return rc;
    TA_LAUNCH("partition_tail", stream, (partition_tail_kernel<U>), dim3(stride_grid(n)), dim3(256),
              static_cast<U*>(out_true), (const U*)parked, n, (const uint64_t*)d_num);
    TA_CHECK_LAUNCH();
    return 0;
  });
}

}  // namespace ta

TA_EXPORT int thrust_amd_copy_if(void* temp, size_t* temp_bytes, const void* in, const void* stencil,
                                 void* out, uint64_t* d_num_selected, uint64_t n, size_t item_bytes,
                                 int stencil_dtype, int cmp, const void* threshold, void* stream) {
  return ta::select_by_predicate(temp, temp_bytes, in, stencil, out, nullptr, d_num_selected, n,
                                 item_bytes, stencil_dtype, cmp, threshold, false, (hipStream_t)stream);
}

TA_EXPORT int thrust_amd_partition_copy(void* temp, size_t* temp_bytes, const void* in,
                                        const void* stencil, void* out_true, void* out_false,
                                        uint64_t* d_num_true, uint64_t n, size_t item_bytes,
                                        int stencil_dtype, int cmp, const void* threshold,
                                        void* stream) {
  if (temp && n && !out_false) return (int)hipErrorInvalidValue;
  return ta::select_by_predicate(temp, temp_bytes, in, stencil, out_true, out_false, d_num_true, n,
                                 item_bytes, stencil_dtype, cmp, threshold, false, (hipStream_t)stream);
}

TA_EXPORT int thrust_amd_stable_partition(void* temp, size_t* temp_bytes, void* data,
                                          const void* stencil, uint64_t* d_num_true, uint64_t n,
                                          size_t item_bytes, int stencil_dtype, int cmp,
                                          const void* threshold, void* stream) {
  return ta::select_by_predicate(temp, temp_bytes, data, stencil, data, nullptr, d_num_true, n,
                                 item_bytes, stencil_dtype, cmp, threshold, true, (hipStream_t)stream);
}

TA_EXPORT int thrust_amd_unique_by_key(void* temp, size_t* temp_bytes, const void* keys_in,
                                       const void* values_in, void* keys_out, void* values_out,
                                       uint64_t* d_num_out, uint64_t n, int key_dtype,
                                       size_t value_bytes, void* stream) {
  using namespace ta;
  if (!temp_bytes || !valid_dtype(key_dtype)) return (int)hipErrorInvalidValue;
  const bool has_values = values_in != nullptr || values_out != nullptr || value_bytes != 0;
  if (has_values && !valid_item_bytes(value_bytes)) return (int)hipErrorInvalidValue;
  return with_dtype(key_dtype, [&](auto tt) {
    using T = typename decltype(tt)::type;
    const SelectTemp lay = select_layout<T>(n, 0);
    if (!temp) {
      *temp_bytes = lay.total;
      return 0;
    }
    if (*temp_bytes < lay.total || !d_num_out || (n && (!keys_in || !keys_out)))
      return (int)hipErrorInvalidValue;
    if (has_values && n && (!values_in || !values_out)) return (int)hipErrorInvalidValue;
    char* base = static_cast<char*>(temp);
    if (!has_values) {
      SelectArgs<T, uint32_t> a{};
      a.tested = static_cast<const T*>(keys_in);
      a.tested_true = static_cast<T*>(keys_out);
      a.d_num_true = d_num_out;
      a.n = n;
      return select_launch<T, uint32_t, FLAG_HEAD, false>(base, lay, a, (hipStream_t)stream);
    }
    return with_item_bytes(value_bytes, [&](auto ut) {
      using U = typename decltype(ut)::type;
      SelectArgs<T, U> a{};
      a.tested = static_cast<const T*>(keys_in);
      a.payload = static_cast<const U*>(values_in);
      a.tested_true = static_cast<T*>(keys_out);
      a.payload_true = static_cast<U*>(values_out);
      a.d_num_true = d_num_out;
      a.n = n;
      return select_launch<T, U, FLAG_HEAD, true>(base, lay, a, (hipStream_t)stream);
    });
  });
}

TA_EXPORT int thrust_amd_unique(void* temp, size_t* temp_bytes, const void* in, void* out,
                                uint64_t* d_num_out, uint64_t n, int dtype, void* stream) {
  return thrust_amd_unique_by_key(temp, temp_bytes, in, nullptr, out, nullptr, d_num_out, n, dtype, 0,
                                  stream);
}
