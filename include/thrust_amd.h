/*
 * thrust_amd.h -- C ABI of the MI355X (gfx950) device system for the Thrust API.
 *
 * Every compute entry point follows the two-phase temporary-storage protocol the
 * reference's CUDA device system uses for its `doit_step` functions
 * (thrust/system/cuda/detail/reduce.h:689-848, sort.h:1149-1269, copy_if.h:602-690,
 * merge.h:676-782):
 *
 *   size_t bytes = 0;
 *   fn(NULL, &bytes, ...);          // size query: writes the bytes needed, launches nothing
 *   fn(temp, &bytes, ...);          // run: enqueues kernels on `stream` and returns
 *
 * Rules that hold for all of them:
 *   - The caller owns every buffer.  Entry points never allocate, free or synchronise.
 *   - All data pointers are DEVICE pointers unless a parameter is documented as a host
 *     pointer (`init`, `threshold`: one scalar of the stated dtype, read during the call).
 *   - Scalar results (`d_out`, `d_num_*`) are written to caller-supplied device memory;
 *     the caller copies them to the host after synchronising the stream.
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream).
 *   - The return value is a hipError_t as int; 0 means success.  No exception crosses
 *     the boundary and nothing aborts.
 *   - n == 0 is legal everywhere.
 *   - Calls are re-entrant and thread-safe as long as they use distinct temp buffers.
 *   - `temp` must be 256-byte aligned (anything from hipMalloc / thrust_amd_malloc is).
 */
#ifndef THRUST_AMD_H
#define THRUST_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define THRUST_AMD_VERSION 100 /* major*100 + minor */

/* Element types understood across the boundary. */
typedef enum thrust_amd_dtype {
  THRUST_AMD_I8 = 0,
  THRUST_AMD_U8 = 1,
  THRUST_AMD_I16 = 2,
  THRUST_AMD_U16 = 3,
  THRUST_AMD_I32 = 4,
  THRUST_AMD_U32 = 5,
  THRUST_AMD_I64 = 6,
  THRUST_AMD_U64 = 7,
  THRUST_AMD_F32 = 8,
  THRUST_AMD_F64 = 9,
  THRUST_AMD_DTYPE_COUNT = 10
} thrust_amd_dtype;

/* Binary operators: the closed set the front end maps thrust::plus / minimum / maximum
 * (and their <void> forms) to.  Integer PLUS wraps modulo 2^bits, which is what the
 * reference's accumulator does (thrust/system/detail/generic/reduce.inl:40-53). */
typedef enum thrust_amd_binop {
  THRUST_AMD_PLUS = 0,
  THRUST_AMD_MIN = 1,
  THRUST_AMD_MAX = 2,
  THRUST_AMD_BINOP_COUNT = 3
} thrust_amd_binop;

/* Unary predicates `x CMP threshold` (threshold has the dtype of the tested array).
 * NONZERO is the reference's default "stencil element converted to bool".  Any code may be
 * or-ed with THRUST_AMD_CMP_NOT: the predicate is then !(x CMP threshold), the logical
 * negation that remove_if applies (thrust/system/cuda/detail/remove.h:40-66 wraps the
 * predicate in not1).  That is not the complementary comparison for floating point: a NaN
 * fails `x < t` and `x >= t` alike, and passes !(x < t). */
typedef enum thrust_amd_cmp {
  THRUST_AMD_LT = 0,
  THRUST_AMD_LE = 1,
  THRUST_AMD_GT = 2,
  THRUST_AMD_GE = 3,
  THRUST_AMD_EQ = 4,
  THRUST_AMD_NE = 5,
  THRUST_AMD_NONZERO = 6,
  THRUST_AMD_CMP_COUNT = 7,
  THRUST_AMD_CMP_NOT = 0x100
} thrust_amd_cmp;

/* Unary transforms applied to every input element by the transform_* entry points: the
 * closed set the front end maps thrust::identity / negate / square to
 * (thrust/functional.h:523-600, 1224-1240).  Integers negate and square modulo 2^bits. */
typedef enum thrust_amd_unary {
  THRUST_AMD_IDENTITY = 0,
  THRUST_AMD_NEGATE = 1,
  THRUST_AMD_SQUARE = 2,
  THRUST_AMD_UNARY_COUNT = 3
} thrust_amd_unary;

/* The four set operations on sorted ranges (multiset semantics,
 * thrust/system/detail/sequential/set_operations.h:42-215). */
typedef enum thrust_amd_set_op {
  THRUST_AMD_SET_DIFFERENCE = 0,
  THRUST_AMD_SET_INTERSECTION = 1,
  THRUST_AMD_SET_SYMMETRIC_DIFFERENCE = 2,
  THRUST_AMD_SET_UNION = 3,
  THRUST_AMD_SET_OP_COUNT = 4
} thrust_amd_set_op;

typedef enum thrust_amd_memcpy_kind {
  THRUST_AMD_H2D = 1,
  THRUST_AMD_D2H = 2,
  THRUST_AMD_D2D = 3
} thrust_amd_memcpy_kind;

/* ------------------------------------------------------------------ library */

/* Library version (THRUST_AMD_VERSION of the build). */
int thrust_amd_version(void);

/* Static, NUL-terminated description of a status code returned by any entry point.
 * Replaces thrust::system::cuda_category().message() (thrust/system/cuda/detail/error.inl). */
const char* thrust_amd_error_string(int status);

/* Size in bytes of one element of `dtype`, 0 for an unknown code. */
size_t thrust_amd_dtype_size(int dtype);

/* ------------------------------------------------------------- memory model */

/* Device allocation / release.  Replace cuda_cub::malloc / cuda_cub::free
 * (thrust/system/cuda/detail/malloc_and_free.h:51-100).  bytes == 0 yields *ptr = NULL. */
int thrust_amd_malloc(void** ptr, size_t bytes);
int thrust_amd_free(void* ptr);

/* Universal memory: one pointer that host code and kernels both dereference.  Replaces the
 * managed allocation behind thrust::universal_vector (thrust/system/cuda/memory_resource.h:
 * 40-110, universal_memory_resource over cudaMallocManaged).  Here it is pinned host memory
 * mapped into the device's address space: nothing migrates, device accesses cross the host
 * link.  Any entry point takes such a pointer where it takes device memory. */
int thrust_amd_malloc_universal(void** ptr, size_t bytes);
int thrust_amd_free_universal(void* ptr);

/* Copy between host and device or device and device, ordered on `stream`; the H2D/D2H
 * forms return after the copy has completed (pageable host memory), the D2D form is
 * asynchronous.  Replaces cuda_cub::trivial_copy_{to,from}_device / trivial_copy_device_to_device
 * (thrust/system/cuda/detail/util.h:107-162) behind copy_cross_system.h:50-200. */
int thrust_amd_memcpy(void* dst, const void* src, size_t bytes, int kind, void* stream);

/* Block until all work enqueued on `stream` has finished.  Replaces
 * cuda_cub::synchronize (thrust/system/cuda/detail/util.h:75-104). */
int thrust_amd_stream_synchronize(void* stream);

/* out[i] = (out_dtype)in[i] with the conversions of C++ (floating point to integer truncates
 * toward zero).  The front end uses it where the reference's algorithms mix types: the
 * accumulator of reduce and exclusive_scan has the type of init, that of inclusive_scan the
 * input's type, and results are converted to the output's element type
 * (thrust/system/detail/generic/reduce.inl:35-53, thrust/system/cuda/detail/scan.h:76-122;
 * testing/reduce.cu:99-129, testing/scan.cu:236-295).  in and out must not overlap unless
 * they are the same address and the types have the same size. */
int thrust_amd_convert(const void* in, int in_dtype, void* out, int out_dtype, uint64_t n,
                       void* stream);

/* out[i] = (T)(init + step * (T)i) for i in [0, n), T the element type named by dtype; init
 * and step point at host values of that type.  Replaces thrust::sequence -> thrust::tabulate
 * with compute_sequence_value (thrust/system/detail/generic/sequence.inl:56-85) for arrays of
 * arithmetic elements, so that code compiled by a plain host compiler can fill its inputs. */
int thrust_amd_sequence(void* out, uint64_t n, int dtype, const void* init, const void* step,
                        void* stream);

/* Streams and events for callers that overlap work (the asynchronous algorithms of the
 * front end).  A stream created here is independent of the null stream; an event is
 * recorded on one stream and another stream can be made to wait for it without blocking
 * the host.  *done = 1 when everything enqueued on the stream has finished.  Streams keep
 * the default priority.  Replace the unique_stream / event machinery of
 * thrust/system/cuda/detail/future.inl:60-260 (cudaStreamCreateWithFlags, cudaEventRecord,
 * cudaStreamWaitEvent, cudaStreamQuery). */
int thrust_amd_stream_create(void** stream);
int thrust_amd_stream_destroy(void* stream);
int thrust_amd_stream_query(void* stream, int* done);
int thrust_amd_event_create(void** event);
int thrust_amd_event_record(void* event, void* stream);
int thrust_amd_stream_wait_event(void* stream, void* event);
int thrust_amd_event_destroy(void* event);

/* Fill n elements of `elem_bytes` (1, 2, 4 or 8) with the host value *value.  Replaces
 * cuda_cub::fill_n (thrust/system/cuda/detail/fill.h) as used by
 * device_vector(n, value) (thrust/detail/vector_base.inl:214-234). */
int thrust_amd_fill(void* dst, uint64_t n, size_t elem_bytes, const void* value, void* stream);

/* Temporary-storage arena: a size-bucketed cache of device blocks, so that the blocking
 * thrust:: front end performs no hipMalloc in steady state.  `acquire` returns a block
 * of at least `bytes`, 256-byte aligned; `release` returns it to the cache once the
 * work enqueued so far on `stream` may be assumed ordered before its next use: `release`
 * records an event on `stream`, and the next `acquire` of that block makes its own stream
 * wait for the event on the device (the host does not block).  The arena keeps the event,
 * never the stream, so a stream may be destroyed while blocks released on it are cached.
 * Blocks are cached per device (the device current at `acquire`); the cache itself is one
 * per process and thread-safe.  `trim` frees every cached block.  Replaces temporary_array<uint8_t,Derived> over
 * get_temporary_buffer (thrust/detail/temporary_array.inl:62-140,
 * thrust/system/detail/generic/temporary_buffer.inl:33-47). */
int thrust_amd_temp_acquire(void** ptr, size_t bytes, void* stream);
int thrust_amd_temp_release(void* ptr, void* stream);
int thrust_amd_temp_trim(void);
/* Bytes currently held by the arena (cached + handed out). */
size_t thrust_amd_temp_bytes_held(void);

/* Per-kernel timing, a debugging aid in the place of the reference's THRUST_DEBUG_SYNC
 * launch log (thrust/system/cuda/config.h:65-69, core/agent_launcher.h:518-535).  While
 * enabled, every kernel the library launches is bracketed by two events on its stream.
 * `collect` waits for the recorded events, writes one line "label launches total_ms" per
 * kernel label into text (NUL-terminated, truncated to capacity; *needed = full size) and
 * forgets them.  Not meant to be left on: it creates two events per launch. */
int thrust_amd_profile_enable(int on);
int thrust_amd_profile_collect(char* text, size_t capacity, size_t* needed);

/* ------------------------------------------------------------------- reduce */

/* *d_out = init OP in[0] OP ... OP in[n-1]; accumulator type = dtype.
 * `init` is a host pointer to one dtype element.  d_out: one dtype element on device.
 * Replaces cuda_cub::detail::reduce_n_impl -> cub::DispatchReduce::Dispatch
 * (thrust/system/cuda/detail/reduce.h:927-1000). */
int thrust_amd_reduce(void* temp, size_t* temp_bytes, const void* in, uint64_t n, int dtype,
                      int op, const void* init, void* d_out, void* stream);

/* *d_count (uint64 on device) = number of elements with (in[i] CMP *threshold); cmp is a
 * thrust_amd_cmp code, `threshold` a host pointer to one dtype element (ignored for
 * THRUST_AMD_NONZERO).
 * Replaces cuda_cub::count_if -> reduce_n over a 0/1 transform
 * (thrust/system/cuda/detail/count.h:43-62; generic form
 * thrust/system/detail/generic/count.inl:64-74). */
int thrust_amd_count_if(void* temp, size_t* temp_bytes, const void* in, uint64_t n, int dtype,
                        int cmp, const void* threshold, uint64_t* d_count, void* stream);

/* *d_out = init + a[0]*b[0] + ... + a[n-1]*b[n-1]; products and sums are made in dtype
 * (integers wrap modulo 2^bits).  `init` is a host pointer to one dtype element.
 * Replaces cuda_cub::inner_product -> transform_reduce over the zipped ranges
 * (thrust/system/cuda/detail/inner_product.h:46-70; generic form
 * thrust/system/detail/generic/inner_product.inl:33-65). */
int thrust_amd_inner_product(void* temp, size_t* temp_bytes, const void* a, const void* b,
                             uint64_t n, int dtype, const void* init, void* d_out, void* stream);

/* *d_out = init OP f(in[0]) OP ... OP f(in[n-1]) with f a thrust_amd_unary code; f's result
 * and the accumulator have type dtype.  `init` is a host pointer to one dtype element.
 * Replaces cuda_cub::transform_reduce -> reduce_n over a transform iterator
 * (thrust/system/cuda/detail/transform_reduce.h:39-64; generic form
 * thrust/system/detail/generic/transform_reduce.inl:30-48). */
int thrust_amd_transform_reduce(void* temp, size_t* temp_bytes, const void* in, uint64_t n,
                                int dtype, int unary, int op, const void* init, void* d_out,
                                void* stream);

/* --------------------------------------------------------------------- scan */

/* out[i] = in[0] OP ... OP in[i]; accumulator type = dtype; out == in allowed.
 * Replaces cuda_cub::inclusive_scan_n -> cub::DispatchScan
 * (thrust/system/cuda/detail/scan.h:55-122). */
int thrust_amd_inclusive_scan(void* temp, size_t* temp_bytes, const void* in, void* out,
                              uint64_t n, int dtype, int op, void* stream);

/* thrust_amd_inclusive_scan for callers that cannot allocate (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc): same result, no temporary storage
 * argument.  It has no counterpart in the reference.  The tile descriptors live in a fixed
 * 1 MiB array inside the library's device image (one copy per GPU, held until the process
 * ends); the call performs no hipMalloc / hipFree.  The array is all zero when the library is
 * loaded and the scan kernel clears what it used before it ends, so the call is ONE kernel
 * launch (the entry point with temporary storage needs a clearing launch first).
 * n is limited by that array: up to 131040 tiles (about 6.4e9 elements of 4 bytes or less,
 * 1.6e9 of 8 bytes); a larger n returns hipErrorInvalidValue and launches nothing.  Every
 * call on a GPU shares that GPU's array.  The library orders such calls itself: each call's
 * stream first waits (on the device) for an event recorded behind the previous call on that GPU,
 * whatever stream or host thread made it.  A stream under capture is left out of that ordering:
 * replays of a graph that holds this call must not overlap other calls of it on the same GPU.
 * The first call on a GPU also looks up the array's address and creates that event (under the
 * relaxed capture mode, should the calling thread be capturing). */
int thrust_amd_inclusive_scan_static(const void* in, void* out, uint64_t n, int dtype, int op,
                                     void* stream);

/* out[0] = init, out[i] = init OP in[0] OP ... OP in[i-1]; out == in allowed.
 * `init` is a host pointer to one dtype element.
 * Replaces cuda_cub::exclusive_scan_n (thrust/system/cuda/detail/scan.h:132-200). */
int thrust_amd_exclusive_scan(void* temp, size_t* temp_bytes, const void* in, void* out,
                              uint64_t n, int dtype, int op, const void* init, void* stream);

/* The two scans above over f(in[i]) instead of in[i], f a thrust_amd_unary code with result
 * type dtype; out == in allowed.
 * Replace cuda_cub::transform_inclusive_scan / transform_exclusive_scan -> the scans over a
 * transform iterator (thrust/system/cuda/detail/transform_scan.h:39-115; generic forms
 * thrust/system/detail/generic/transform_scan.inl:37-97). */
int thrust_amd_transform_inclusive_scan(void* temp, size_t* temp_bytes, const void* in, void* out,
                                        uint64_t n, int dtype, int unary, int op, void* stream);
int thrust_amd_transform_exclusive_scan(void* temp, size_t* temp_bytes, const void* in, void* out,
                                        uint64_t n, int dtype, int unary, int op, const void* init,
                                        void* stream);

/* Segmented scans: a segment is a run of equal consecutive keys (compared like
 * reduce_by_key: integers by value, floats with ==).  out[i] = the OP-fold of the segment's
 * values up to and including i.  out may alias values.  Accumulator = value_dtype;
 * floating-point folds use a tree order inside a segment.
 * Replaces cuda_cub::inclusive_scan_by_key (thrust/system/cuda/detail/scan_by_key.h:795-880;
 * generic form thrust/system/detail/generic/scan_by_key.inl:96-135). */
int thrust_amd_inclusive_scan_by_key(void* temp, size_t* temp_bytes, const void* keys,
                                     const void* values, void* out, uint64_t n, int key_dtype,
                                     int value_dtype, int op, void* stream);

/* out[i] = *init at the first element of a segment, else init OP (the segment's values
 * before i).  `init` is a host pointer to one value_dtype element.  out may alias values.
 * Replaces cuda_cub::exclusive_scan_by_key (thrust/system/cuda/detail/scan_by_key.h:885-1000;
 * generic form thrust/system/detail/generic/scan_by_key.inl:190-238). */
int thrust_amd_exclusive_scan_by_key(void* temp, size_t* temp_bytes, const void* keys,
                                     const void* values, void* out, uint64_t n, int key_dtype,
                                     int value_dtype, int op, const void* init, void* stream);

/* --------------------------------------------------------------------- sort */

/* Stable in-place sort of n keys by the total order of their radix encoding:
 * unsigned = value, signed = sign bit flipped, float = IEEE bits ^ (-(bits>>31) | signbit)
 * (-0.0 before +0.0, NaNs by bit pattern), the reference's encoders
 * (thrust/system/detail/sequential/stable_radix_sort.inl:41-138).  Only key bits
 * [begin_bit, end_bit) take part (0 and 8*sizeof(key) sort fully).  descending != 0
 * yields the order thrust::greater<Key> gives, still stable.  n <= 2^32 - 1 per call
 * (hipErrorInvalidValue beyond).
 * Replaces cuda_cub::__radix_sort::dispatch -> cub::DeviceRadixSort::SortKeys[Descending]
 * (thrust/system/cuda/detail/sort.h:1326-1429,1438-1508). */
int thrust_amd_sort_keys(void* temp, size_t* temp_bytes, void* keys, uint64_t n, int key_dtype,
                         int descending, int begin_bit, int end_bit, void* stream);

/* Same for key-value pairs; values are opaque items of value_bytes (1, 2, 4 or 8) that
 * travel with their key.  Replaces cub::DeviceRadixSort::SortPairs[Descending]
 * (thrust/system/cuda/detail/sort.h:1383-1427). */
int thrust_amd_sort_pairs(void* temp, size_t* temp_bytes, void* keys, void* values, uint64_t n,
                          int key_dtype, size_t value_bytes, int descending, int begin_bit,
                          int end_bit, void* stream);

/* Stable comparison sort (merge sort) by operator< (descending != 0: operator>), the path
 * thrust::sort takes when the comparator is not thrust::less / thrust::greater of an
 * arithmetic key.  The order is the comparison's, not the bit pattern's: for floating-point
 * keys -0.0 and +0.0 are equivalent and keep their input order (the radix entry points put
 * -0.0 first); NaN keys are outside a strict weak order and not supported.  Same temp
 * convention; n * (key + value) bytes of temp plus 8 bytes per 4096 elements.
 * The kernels are the templates of include/thrust/system/hip/detail/merge_sort_kernels.h,
 * which a translation unit compiled with hipcc instantiates for its own comparators.
 * Replaces cuda_cub::__merge_sort::merge_sort (thrust/system/cuda/detail/sort.h:1278-1322;
 * BlockSortAgent :235-633, PartitionAgent :638-694, MergeAgent :701-1138). */
int thrust_amd_merge_sort_keys(void* temp, size_t* temp_bytes, void* keys, uint64_t n, int key_dtype,
                               int descending, void* stream);
int thrust_amd_merge_sort_pairs(void* temp, size_t* temp_bytes, void* keys, void* values, uint64_t n,
                                int key_dtype, size_t value_bytes, int descending, void* stream);

/* ---------------------------------------------------------- set operations */

/* out = a OP b for two ranges sorted by operator< (descending != 0: by operator>), OP a
 * thrust_amd_set_op code.  A key that occurs m times in a and n times in b appears
 * max(m-n,0) times (difference, the last copies of a), min(m,n) times (intersection, the
 * first copies of a), |m-n| times (symmetric difference, the last copies of the longer
 * side) or max(m,n) times (union: all of a, then the last n-m copies of b); the result is
 * sorted and stable.  *d_num_out (uint64 on device) receives its length; out must hold
 * na + nb elements for union and symmetric difference, na for difference, min(na, nb) for
 * intersection, and must not overlap a or b.  na + nb < 2^43.
 * Replaces cuda_cub::set_difference / set_intersection / set_symmetric_difference /
 * set_union (thrust/system/cuda/detail/set_operations.h:1480-1960). */
int thrust_amd_set_operation(void* temp, size_t* temp_bytes, int op, const void* a, uint64_t na,
                             const void* b, uint64_t nb, void* out, uint64_t* d_num_out, int dtype,
                             int descending, void* stream);

/* Same on keys, with one value (opaque item of value_bytes = 1, 2, 4 or 8) travelling with
 * every kept key from the range the key came from.  values_b is read only by union and
 * symmetric difference and may be NULL otherwise.
 * Replaces the *_by_key forms (thrust/system/cuda/detail/set_operations.h:1480-1960). */
int thrust_amd_set_operation_by_key(void* temp, size_t* temp_bytes, int op, const void* keys_a,
                                    uint64_t na, const void* keys_b, uint64_t nb,
                                    const void* values_a, const void* values_b, void* keys_out,
                                    void* values_out, uint64_t* d_num_out, int key_dtype,
                                    size_t value_bytes, int descending, void* stream);

/* ----------------------------------------------------- selection / partition */

/* Stable compaction: copies in[i] (items of item_bytes = 1, 2, 4 or 8) to out, in order,
 * for every i whose tested element satisfies `tested CMP *threshold`; the tested
 * element is stencil[i] (dtype stencil_dtype) or, when stencil == NULL, in[i] itself
 * (then stencil_dtype is the dtype of `in`).  *d_num_selected (uint64 on device)
 * receives the count.  out may alias in.
 * Replaces cuda_cub::__copy_if::copy_if (thrust/system/cuda/detail/copy_if.h:699-773). */
int thrust_amd_copy_if(void* temp, size_t* temp_bytes, const void* in, const void* stencil,
                       void* out, uint64_t* d_num_selected, uint64_t n, size_t item_bytes,
                       int stencil_dtype, int cmp, const void* threshold, void* stream);

/* Stable two-way split: selected items go to out_true, the others to out_false, both
 * in their original order; *d_num_true (uint64 on device) receives the number selected.
 * out_true may alias in.
 * Replaces cuda_cub::__partition::partition with two outputs
 * (thrust/system/cuda/detail/partition.h:612-795, stable_partition_copy :925-1010). */
int thrust_amd_partition_copy(void* temp, size_t* temp_bytes, const void* in,
                              const void* stencil, void* out_true, void* out_false,
                              uint64_t* d_num_true, uint64_t n, size_t item_bytes,
                              int stencil_dtype, int cmp, const void* threshold, void* stream);

/* In-place stable partition of `data`: selected items first, then the rest, each group
 * in its original order; *d_num_true receives the split point.
 * Replaces cuda_cub::__partition::partition_inplace + the trailing reverse
 * (thrust/system/cuda/detail/partition.h:796-824,1068-1120). */
int thrust_amd_stable_partition(void* temp, size_t* temp_bytes, void* data, const void* stencil,
                                uint64_t* d_num_true, uint64_t n, size_t item_bytes,
                                int stencil_dtype, int cmp, const void* threshold, void* stream);

/* Keeps the first element of every run of equal consecutive elements
 * (run boundary at i where in[i-1] != in[i]; element 0 always kept).  Floating-point
 * keys compare with ==, as thrust::equal_to does.  out may alias in.
 * Replaces cuda_cub::__unique::unique (thrust/system/cuda/detail/unique.h:635-700). */
int thrust_amd_unique(void* temp, size_t* temp_bytes, const void* in, void* out,
                      uint64_t* d_num_out, uint64_t n, int dtype, void* stream);

/* Same on keys, carrying the FIRST value of each run along; values are opaque items of
 * value_bytes (1, 2, 4 or 8).  keys_out / values_out may alias the inputs.
 * Replaces cuda_cub::__unique_by_key::unique_by_key
 * (thrust/system/cuda/detail/unique_by_key.h:732-800). */
int thrust_amd_unique_by_key(void* temp, size_t* temp_bytes, const void* keys_in,
                             const void* values_in, void* keys_out, void* values_out,
                             uint64_t* d_num_out, uint64_t n, int key_dtype, size_t value_bytes,
                             void* stream);

/* For every run of equal consecutive keys writes the run's first key and the OP-fold of
 * its values (accumulator = value_dtype; floating-point sums use a tree order inside a
 * run, so they agree with a left fold to rounding only).  *d_num_runs receives the
 * number of runs.  Outputs must not alias inputs.
 * Replaces cuda_cub::__reduce_by_key::reduce_by_key
 * (thrust/system/cuda/detail/reduce_by_key.h:974-1055). */
int thrust_amd_reduce_by_key(void* temp, size_t* temp_bytes, const void* keys_in,
                             const void* values_in, void* keys_out, void* values_out,
                             uint64_t* d_num_runs, uint64_t n, int key_dtype, int value_dtype,
                             int op, void* stream);

/* -------------------------------------------------------------------- merge */

/* Stable merge of two ranges sorted by operator< of dtype (ascending; by operator> when
 * descending != 0) into out (na + nb elements).  Keys are compared by value: for floats
 * -0.0 and +0.0 are equal.  Ties: every equal element of `a` precedes those of `b`
 * (thrust/system/detail/sequential/merge.inl:56-65).  out must not alias a or b.
 * Replaces cuda_cub::__merge::merge keys-only (thrust/system/cuda/detail/merge.h:785-853). */
int thrust_amd_merge(void* temp, size_t* temp_bytes, const void* a, uint64_t na, const void* b,
                     uint64_t nb, void* out, int dtype, int descending, void* stream);

/* Same with values (opaque items of value_bytes = 1, 2, 4 or 8) travelling with the keys.
 * Replaces cuda_cub::__merge::merge with items (thrust/system/cuda/detail/merge.h:785-853,
 * merge_by_key :930-1010). */
int thrust_amd_merge_by_key(void* temp, size_t* temp_bytes, const void* keys_a, uint64_t na,
                            const void* keys_b, uint64_t nb, const void* values_a,
                            const void* values_b, void* keys_out, void* values_out,
                            int key_dtype, size_t value_bytes, int descending, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* THRUST_AMD_H */
