// Memory model and plumbing of the device system: allocation, copies, synchronisation,
// fill, and the temporary-storage arena.  These are the only entry points that
// allocate or block; every compute entry point works on caller-owned memory.
#include "common.hpp"
#include "dispatch.hpp"
#include "launch.hpp"

#include <atomic>
#include <cstdio>
#include <cstring>
#include <map>
#include <string>
#include <mutex>
#include <vector>

TA_EXPORT int thrust_amd_version(void) { return THRUST_AMD_VERSION; }

TA_EXPORT const char* thrust_amd_error_string(int status) {
  return hipGetErrorString((hipError_t)status);
}

TA_EXPORT size_t thrust_amd_dtype_size(int dtype) {
  switch (dtype) {
    case THRUST_AMD_I8: case THRUST_AMD_U8: return 1;
    case THRUST_AMD_I16: case THRUST_AMD_U16: return 2;
    case THRUST_AMD_I32: case THRUST_AMD_U32: case THRUST_AMD_F32: return 4;
    case THRUST_AMD_I64: case THRUST_AMD_U64: case THRUST_AMD_F64: return 8;
    default: return 0;
  }
}

TA_EXPORT int thrust_amd_malloc(void** ptr, size_t bytes) {
  if (!ptr) return (int)hipErrorInvalidValue;
  *ptr = nullptr;
  if (bytes == 0) return 0;
  hipError_t e = hipMalloc(ptr, bytes);
  if (e != hipSuccess) {
    (void)hipGetLastError();  // an allocation failure must not poison later calls
    *ptr = nullptr;
  }
  return (int)e;
}

TA_EXPORT int thrust_amd_free(void* ptr) {
  if (!ptr) return 0;
  return (int)hipFree(ptr);
}

// Universal memory: pinned host memory that the device addresses directly.  Both sides can
// dereference the same pointer and no page ever migrates or faults.
TA_EXPORT int thrust_amd_malloc_universal(void** ptr, size_t bytes) {
  if (!ptr) return (int)hipErrorInvalidValue;
  *ptr = nullptr;
  if (bytes == 0) return 0;
  hipError_t e = hipHostMalloc(ptr, bytes, hipHostMallocDefault);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    *ptr = nullptr;
  }
  return (int)e;
}

TA_EXPORT int thrust_amd_free_universal(void* ptr) {
  if (!ptr) return 0;
  return (int)hipHostFree(ptr);
}

TA_EXPORT int thrust_amd_memcpy(void* dst, const void* src, size_t bytes, int kind, void* stream) {
  if (bytes == 0) return 0;
  if (!dst || !src) return (int)hipErrorInvalidValue;
  hipStream_t s = (hipStream_t)stream;
  switch (kind) {
    // the runtime resolves the address spaces itself (hipMemcpyDefault), so that universal
    // memory may stand on either side; `kind` keeps deciding whether the call blocks
    case THRUST_AMD_H2D:
    case THRUST_AMD_D2H:
      TA_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDefault, s));
      return (int)hipStreamSynchronize(s);
    case THRUST_AMD_D2D:
      return (int)hipMemcpyAsync(dst, src, bytes, hipMemcpyDefault, s);
    default:
      return (int)hipErrorInvalidValue;
  }
}

TA_EXPORT int thrust_amd_stream_synchronize(void* stream) {
  return (int)hipStreamSynchronize((hipStream_t)stream);
}

TA_EXPORT int thrust_amd_stream_create(void** stream) {
  if (!stream) return (int)hipErrorInvalidValue;
  hipStream_t s = nullptr;
  const hipError_t e = hipStreamCreateWithFlags(&s, hipStreamNonBlocking);
  *stream = (e == hipSuccess) ? (void*)s : nullptr;
  return (int)e;
}

TA_EXPORT int thrust_amd_stream_destroy(void* stream) {
  if (!stream) return 0;
  return (int)hipStreamDestroy((hipStream_t)stream);
}

TA_EXPORT int thrust_amd_stream_query(void* stream, int* done) {
  if (!done) return (int)hipErrorInvalidValue;
  const hipError_t e = hipStreamQuery((hipStream_t)stream);
  if (e == hipErrorNotReady) {
    (void)hipGetLastError();  // "not ready" is an answer, not a failure to leave behind
    *done = 0;
    return 0;
  }
  *done = (e == hipSuccess) ? 1 : 0;
  return (int)e;
}

TA_EXPORT int thrust_amd_event_create(void** event) {
  if (!event) return (int)hipErrorInvalidValue;
  hipEvent_t ev = nullptr;
  const hipError_t e = hipEventCreateWithFlags(&ev, hipEventDisableTiming);
  *event = (e == hipSuccess) ? (void*)ev : nullptr;
  return (int)e;
}

TA_EXPORT int thrust_amd_event_record(void* event, void* stream) {
  if (!event) return (int)hipErrorInvalidValue;
  return (int)hipEventRecord((hipEvent_t)event, (hipStream_t)stream);
}

TA_EXPORT int thrust_amd_stream_wait_event(void* stream, void* event) {
  if (!event) return (int)hipErrorInvalidValue;
  return (int)hipStreamWaitEvent((hipStream_t)stream, (hipEvent_t)event, 0);
}

TA_EXPORT int thrust_amd_event_destroy(void* event) {
  if (!event) return 0;
  return (int)hipEventDestroy((hipEvent_t)event);
}

namespace ta {

template <typename U>
__global__ __launch_bounds__(256) void fill_kernel(U* __restrict__ dst, uint64_t n, U value) {
  constexpr int VEC = Vec16<U>::N;
  const uint64_t vecs = n / VEC;
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  const uint64_t tid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  // dst is element-aligned only; peel to the first 16-byte boundary.
  const uint64_t mis = (reinterpret_cast<uintptr_t>(dst) & 15u) / sizeof(U);
  const uint64_t head = mis ? ((VEC - mis) < n ? (VEC - mis) : n) : 0;
  if (tid < head) dst[tid] = value;
  U* body = dst + head;
  const uint64_t body_vecs = (n - head) / VEC;
  Vec16<U> v;
#pragma unroll
  for (int i = 0; i < VEC; ++i) v.v[i] = value;
  for (uint64_t i = tid; i < body_vecs; i += stride) reinterpret_cast<Vec16<U>*>(body)[i] = v;
  const uint64_t tail_begin = head + body_vecs * VEC;
  if (tail_begin + tid < n) dst[tail_begin + tid] = value;  // < VEC elements, grid has >= 256 threads
  (void)vecs;
}

}  // namespace ta

TA_EXPORT int thrust_amd_fill(void* dst, uint64_t n, size_t elem_bytes, const void* value,
                               void* stream) {
  using namespace ta;
  if (!valid_item_bytes(elem_bytes)) return (int)hipErrorInvalidValue;
  if (n == 0) return 0;
  if (!dst || !value) return (int)hipErrorInvalidValue;
  return with_item_bytes(elem_bytes, [&](auto tt) {
    using U = typename decltype(tt)::type;
    U v;
    __builtin_memcpy(&v, value, sizeof(U));
    const uint64_t vecs = n / Vec16<U>::N + 1;
    uint64_t blocks = (vecs + 255) / 256;
    const uint64_t cap = (uint64_t)NUM_CU * 16;
    if (blocks > cap) blocks = cap;
    TA_LAUNCH("fill", (hipStream_t)stream, (fill_kernel<U>), dim3((uint32_t)blocks), dim3(256), static_cast<U*>(dst), n, v);
    TA_CHECK_LAUNCH();
    return 0;
  });
}

namespace ta {
template <typename In, typename Out>
__global__ __launch_bounds__(256) void convert_kernel(const In* in, Out* out, uint64_t n) {
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) out[i] = static_cast<Out>(in[i]);
}
}  // namespace ta

TA_EXPORT int thrust_amd_convert(const void* in, int in_dtype, void* out, int out_dtype, uint64_t n,
                                 void* stream) {
  using namespace ta;
  if (!valid_dtype(in_dtype) || !valid_dtype(out_dtype)) return (int)hipErrorInvalidValue;
  if (n == 0) return 0;
  if (!in || !out) return (int)hipErrorInvalidValue;
  return with_dtype(in_dtype, [&](auto it) {
    using In = typename decltype(it)::type;
    return with_dtype(out_dtype, [&](auto ot) {
      using Out = typename decltype(ot)::type;
      uint64_t blocks = (n + 255) / 256;
      const uint64_t cap = (uint64_t)1 << 20;  // one element per lane up to 2^28; short workgroups keep more requests in flight
      if (blocks > cap) blocks = cap;
      TA_LAUNCH("convert", (hipStream_t)stream, (convert_kernel<In, Out>), dim3((uint32_t)blocks), dim3(256),
                static_cast<const In*>(in), static_cast<Out*>(out), n);
      TA_CHECK_LAUNCH();
      return 0;
    });
  });
}

namespace ta {
// The product is rounded before the sum, as in the reference's host back ends (no fused
// multiply-add), so that floating-point sequences agree with them bit for bit.
template <typename T>
__global__ __launch_bounds__(256) void sequence_kernel(T* out, uint64_t n, T init, T step) {
#pragma clang fp contract(off)
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
    out[i] = static_cast<T>(init + step * static_cast<T>(i));
}
}  // namespace ta

TA_EXPORT int thrust_amd_sequence(void* out, uint64_t n, int dtype, const void* init, const void* step,
                                  void* stream) {
  using namespace ta;
  if (!valid_dtype(dtype)) return (int)hipErrorInvalidValue;
  if (n == 0) return 0;
  if (!out || !init || !step) return (int)hipErrorInvalidValue;
  return with_dtype(dtype, [&](auto tt) {
    using T = typename decltype(tt)::type;
    T first, by;
    __builtin_memcpy(&first, init, sizeof(T));
    __builtin_memcpy(&by, step, sizeof(T));
    uint64_t blocks = (n + 255) / 256;
    const uint64_t cap = (uint64_t)1 << 20;
    if (blocks > cap) blocks = cap;
    TA_LAUNCH("sequence", (hipStream_t)stream, (sequence_kernel<T>), dim3((uint32_t)blocks), dim3(256),
              static_cast<T*>(out), n, first, by);
    TA_CHECK_LAUNCH();
    return 0;
  });
}

// ------------------------------------------------------------------ temp arena
// Blocks are rounded up to size classes (powers of two from 4 KiB to 64 MiB, then
// multiples of 64 MiB -- a 2^28-key radix sort needs ~1.2 GiB and must not round to
// 2 GiB) and cached per device.  Every block owns one event.  Releasing a block records
// that event on the releasing stream; handing the block out again makes the acquiring
// stream wait for the event on the device (no host blocking).  The arena never keeps a
// stream handle to call into later: the stream a block was released on may be destroyed at
// any time, the event stays valid.  The handle is kept only as a tag, compared and never
// used, to prefer a block last used on the same stream.
namespace ta {

struct ArenaBlock {
  void* ptr;
  size_t bytes;
  int device;
  hipEvent_t released;        // recorded at the last release; null before the first one
  const void* released_tag;   // value of the releasing stream handle (identity only)
};

struct Arena {
  std::mutex mu;
  std::multimap<std::pair<int, size_t>, ArenaBlock> free_blocks;  // by (device, size class)
  std::map<void*, ArenaBlock> live;                                // handed out
  size_t held = 0;
};

static Arena& arena() {
  static Arena* a = new Arena;  // leaked on purpose: no hipFree during static destruction
  return *a;
}

static size_t size_class(size_t bytes) {
  const size_t lo = 4096, hi = (size_t)64 << 20;
  if (bytes <= lo) return lo;
  if (bytes <= hi) {
    size_t c = lo;
    while (c < bytes) c <<= 1;
    return c;
  }
  return align_up(bytes, hi);
}

static int trim_device(int device, bool all_devices) {
  Arena& a = arena();
  std::vector<ArenaBlock> victims;
  {
    std::lock_guard<std::mutex> g(a.mu);
    for (auto it = a.free_blocks.begin(); it != a.free_blocks.end();) {
      if (all_devices || it->second.device == device) {
        victims.push_back(it->second);
        a.held -= it->second.bytes;
        it = a.free_blocks.erase(it);
      } else {
        ++it;
      }
    }
  }
  int rc = 0;
  for (auto& b : victims) {
    hipError_t e = hipSuccess;
    if (b.released) {
      e = hipEventSynchronize(b.released);  // the last user of the block has finished
      (void)hipEventDestroy(b.released);
    }
    const hipError_t f = hipFree(b.ptr);
    if (e == hipSuccess) e = f;
    if (e != hipSuccess && rc == 0) rc = (int)e;
  }
  return rc;
}

}  // namespace ta

TA_EXPORT int thrust_amd_temp_acquire(void** ptr, size_t bytes, void* stream) {
  using namespace ta;
  if (!ptr) return (int)hipErrorInvalidValue;
  *ptr = nullptr;
  if (bytes == 0) return 0;
  int device = 0;
  TA_CHECK(hipGetDevice(&device));
  const size_t cls = size_class(bytes);
  Arena& a = arena();
  ArenaBlock blk{nullptr, 0, device, nullptr, nullptr};
  {
    std::lock_guard<std::mutex> g(a.mu);
    auto range = a.free_blocks.equal_range(std::make_pair(device, cls));
    auto pick = range.second;
    for (auto it = range.first; it != range.second; ++it) {
      if (it->second.released_tag == (const void*)stream) { pick = it; break; }
      if (pick == range.second) pick = it;
    }
    if (pick != range.second) {
      blk = pick->second;
      a.free_blocks.erase(pick);
    }
  }
  if (blk.ptr) {
    if (blk.released) {
      // Work enqueued on `stream` from here on starts after the block's last use.  On the
      // releasing stream itself this adds nothing that stream order did not already give.
      const hipError_t e = hipStreamWaitEvent((hipStream_t)stream, blk.released, 0);
      if (e != hipSuccess) {
        std::lock_guard<std::mutex> g(a.mu);  // the block stays cached, not lost
        a.free_blocks.emplace(std::make_pair(device, cls), blk);
        return (int)e;
      }
    }
    {
      std::lock_guard<std::mutex> g(a.mu);
      a.live[blk.ptr] = blk;
    }
    *ptr = blk.ptr;
    return 0;
  }
  void* p = nullptr;
  hipError_t e = hipMalloc(&p, cls);
  if (e != hipSuccess) {
    // Out of memory: give this device's cached blocks back to the driver and try once more.
    (void)hipGetLastError();
    (void)trim_device(device, false);
    e = hipMalloc(&p, cls);
    if (e != hipSuccess) {
      (void)hipGetLastError();
      return (int)e;
    }
  }
  {
    std::lock_guard<std::mutex> g(a.mu);
    a.live[p] = ArenaBlock{p, cls, device, nullptr, nullptr};
    a.held += cls;
  }
  *ptr = p;
  return 0;
}

TA_EXPORT int thrust_amd_temp_release(void* ptr, void* stream) {
  using namespace ta;
  if (!ptr) return 0;
  Arena& a = arena();
  ArenaBlock blk;
  {
    std::lock_guard<std::mutex> g(a.mu);
    auto it = a.live.find(ptr);
    if (it == a.live.end()) return (int)hipErrorInvalidValue;
    blk = it->second;
    a.live.erase(it);
  }
  // Mark the end of the block's use on the releasing stream.  If that cannot be done the
  // stream is drained instead, and the block goes back without an event to wait for.
  hipError_t e = hipSuccess;
  if (!blk.released) e = hipEventCreateWithFlags(&blk.released, hipEventDisableTiming);
  if (e == hipSuccess) e = hipEventRecord(blk.released, (hipStream_t)stream);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    if (blk.released) (void)hipEventDestroy(blk.released);
    blk.released = nullptr;
    e = hipStreamSynchronize((hipStream_t)stream);
  }
  blk.released_tag = (const void*)stream;
  {
    std::lock_guard<std::mutex> g(a.mu);
    a.free_blocks.emplace(std::make_pair(blk.device, blk.bytes), blk);
  }
  return (int)e;
}

TA_EXPORT int thrust_amd_temp_trim(void) { return ta::trim_device(0, true); }

TA_EXPORT size_t thrust_amd_temp_bytes_held(void) {
  using namespace ta;
  Arena& a = arena();
  std::lock_guard<std::mutex> g(a.mu);
  return a.held;
}

// ------------------------------------------------------------------ per-kernel timing
namespace ta {

struct ProfileRecord {
  const char* label;
  hipEvent_t begin, end;
};

struct Profile {
  std::mutex mu;
  std::vector<ProfileRecord> records;
};

static std::atomic<int> g_profile_on{0};
static Profile& profile() {
  static Profile* p = new Profile;
  return *p;
}

bool profile_on() { return g_profile_on.load(std::memory_order_relaxed) != 0; }

hipEvent_t profile_begin(hipStream_t stream) {
  hipEvent_t ev = nullptr;
  if (hipEventCreate(&ev) != hipSuccess) return nullptr;
  if (hipEventRecord(ev, stream) != hipSuccess) {
    (void)hipEventDestroy(ev);
    return nullptr;
  }
  return ev;
}

void profile_end(const char* label, hipStream_t stream, hipEvent_t begin) {
  hipEvent_t ev = nullptr;
  if (hipEventCreate(&ev) != hipSuccess || hipEventRecord(ev, stream) != hipSuccess) {
    if (ev) (void)hipEventDestroy(ev);
    (void)hipEventDestroy(begin);
    return;
  }
  Profile& p = profile();
  std::lock_guard<std::mutex> g(p.mu);
  p.records.push_back(ProfileRecord{label, begin, ev});
}

}  // namespace ta

TA_EXPORT int thrust_amd_profile_enable(int on) {
  ta::g_profile_on.store(on ? 1 : 0);
  return 0;
}

TA_EXPORT int thrust_amd_profile_collect(char* text, size_t capacity, size_t* needed) {
  using namespace ta;
  Profile& p = profile();
  std::vector<ProfileRecord> recs;
  {
    std::lock_guard<std::mutex> g(p.mu);
    recs.swap(p.records);
  }
  // label -> (launches, total ms), in order of first appearance
  std::vector<std::pair<const char*, std::pair<uint64_t, double>>> agg;
  int rc = 0;
  for (auto& r : recs) {
    float ms = 0.f;
    hipError_t e = hipEventSynchronize(r.end);
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, r.begin, r.end);
    if (e != hipSuccess && rc == 0) rc = (int)e;
    (void)hipEventDestroy(r.begin);
    (void)hipEventDestroy(r.end);
    bool found = false;
    for (auto& a : agg)
      if (std::string(a.first) == r.label) {
        a.second.first++;
        a.second.second += ms;
        found = true;
        break;
      }
    if (!found) agg.push_back({r.label, {1, (double)ms}});
  }
  std::string out;
  for (auto& a : agg) {
    char line[160];
    snprintf(line, sizeof line, "%s %llu %.6f\n", a.first, (unsigned long long)a.second.first,
             a.second.second);
    out += line;
  }
  if (needed) *needed = out.size() + 1;
  if (text && capacity) {
    const size_t nbytes = out.size() < capacity - 1 ? out.size() : capacity - 1;
    memcpy(text, out.data(), nbytes);
    text[nbytes] = 0;
  }
  return rc;
}
