/* TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.
 *
 * CPU restatement of the reference's OpenMP / sequential device system (Thrust 1.14.0)
 * for the algorithms the gfx950 library implements.  It exists so that tests can check
 * the device results on a machine where the reference tree is absent, and so that the
 * benchmark can time a CPU baseline.  Only tests, the smoke check and the benchmark's
 * cpu_baseline leg may load it; the library never does.
 *
 * Every function takes HOST pointers and mirrors the argument meaning of the
 * corresponding thrust_amd_* entry point.  Each restated routine cites the reference
 * file:line it follows (paths under the reference tree's thrust/system/).
 *
 * How each function is pinned (nothing here is "parity unpinned"):
 *   - against the literal known-answer vectors of the reference's own unit tests
 *     (tests/golden/known_answers.json),
 *   - against outputs of the real reference built from its sources (oracle/_ref, both
 *     the OMP and the CPP device system) on seeded inputs (tests/golden/ fixtures and, where
 *     oracle/_ref is present, live in tests/test_oracle.py:
 *     test_oracle_matches_live_reference_on_ragged_sizes),
 *   - against independent definitions (numpy cumsum mod 2^k, np.sort(kind="stable"),
 *     brute-force filters, float64 folds) in tests/test_oracle.py.
 */
#include <omp.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include "../include/thrust_amd.h"

#define ORACLE_API __attribute__((visibility("default")))

/* uniform_decomposition (detail/internal/decompose.h:54-107). */
typedef struct {
  long N, intervals, threshold, small_interval, large_interval;
} decomp_t;

static decomp_t decomp_make(long N, long granularity, long max_intervals) {
  decomp_t d;
  d.N = N;
  d.intervals = (N + granularity - 1) / granularity;
  d.threshold = 0;
  d.small_interval = granularity;
  d.large_interval = 0;
  if (d.intervals > max_intervals) {
    d.small_interval = granularity * (d.intervals / max_intervals);
    d.large_interval = d.small_interval + granularity;
    d.threshold = d.intervals % max_intervals;
    d.intervals = max_intervals;
  }
  return d;
}

static void decomp_range(const decomp_t* d, long i, long* begin, long* end) {
  if (i < d->threshold) {
    *begin = d->large_interval * i;
    *end = *begin + d->large_interval;
  } else {
    *begin = d->large_interval * d->threshold + d->small_interval * (i - d->threshold);
    *end = (*begin + d->small_interval < d->N) ? *begin + d->small_interval : d->N;
  }
}

/* Exposed so that tests can pin the decomposition against
 * testing/omp/reduce_intervals.cu:49-78 and testing/decompose.cu. */
ORACLE_API long oracle_decompose(long N, long granularity, long max_intervals, long* begins,
                                 long* ends) {
  decomp_t d = decomp_make(N, granularity, max_intervals);
  for (long i = 0; i < d.intervals; i++) decomp_range(&d, i, begins + i, ends + i);
  return d.intervals;
}

static void reverse_sz(size_t* x, size_t n) {
  for (size_t i = 0; i < n / 2; i++) {
    size_t t = x[i];
    x[i] = x[n - 1 - i];
    x[n - 1 - i] = t;
  }
}

#define T int8_t
#define U uint8_t
#define S i8
#define IS_FLOAT 0
#define IS_SIGNED 1
#include "oracle_type.inc"
#undef T
#undef U
#undef S
#undef IS_SIGNED
#define T uint8_t
#define U uint8_t
#define S u8
#define IS_SIGNED 0
#include "oracle_type.inc"
#undef T
#undef U
#undef S
#undef IS_SIGNED
#define T int16_t
#define U uint16_t
#define S i16
#define IS_SIGNED 1
#include "oracle_type.inc"
#undef T
#undef U
#undef S
#undef IS_SIGNED
#define T uint16_t
#define U uint16_t
#define S u16
#define IS_SIGNED 0
#include "oracle_type.inc"
#undef T
#undef U
#undef S
#undef IS_SIGNED
#define T int32_t
#define U uint32_t
#define S i32
#define IS_SIGNED 1
#include "oracle_type.inc"
#undef T
#undef U
#undef S
#undef IS_SIGNED
#define T uint32_t
#define U uint32_t
#define S u32
#define IS_SIGNED 0
#include "oracle_type.inc"
#undef T
#undef U
#undef S
#undef IS_SIGNED
#define T int64_t
#define U uint64_t
#define S i64
#define IS_SIGNED 1
#include "oracle_type.inc"
#undef T
#undef U
#undef S
#undef IS_SIGNED
#define T uint64_t
#define U uint64_t
#define S u64
#define IS_SIGNED 0
#include "oracle_type.inc"
#undef T
#undef U
#undef S
#undef IS_SIGNED
#undef IS_FLOAT
#define IS_FLOAT 1
#define IS_SIGNED 1
#define T float
#define U uint32_t
#define S f32
#include "oracle_type.inc"
#undef T
#undef U
#undef S
#define T double
#define U uint64_t
#define S f64
#include "oracle_type.inc"
#undef T
#undef U
#undef S

/* Runs STMT with the macro-style token X bound per dtype: DISPATCH(dtype, X, stmt using X(name)). */
#define DISPATCH(dtype, BODY)                                  \
  switch (dtype) {                                             \
    case THRUST_AMD_I8: { BODY(i8, int8_t) } break;            \
    case THRUST_AMD_U8: { BODY(u8, uint8_t) } break;           \
    case THRUST_AMD_I16: { BODY(i16, int16_t) } break;         \
    case THRUST_AMD_U16: { BODY(u16, uint16_t) } break;        \
    case THRUST_AMD_I32: { BODY(i32, int32_t) } break;         \
    case THRUST_AMD_U32: { BODY(u32, uint32_t) } break;        \
    case THRUST_AMD_I64: { BODY(i64, int64_t) } break;         \
    case THRUST_AMD_U64: { BODY(u64, uint64_t) } break;        \
    case THRUST_AMD_F32: { BODY(f32, float) } break;           \
    case THRUST_AMD_F64: { BODY(f64, double) } break;          \
    default: return -1;                                        \
  }

static size_t dtype_size(int dtype) {
  static const size_t sz[10] = {1, 1, 2, 2, 4, 4, 8, 8, 4, 8};
  return (dtype >= 0 && dtype < 10) ? sz[dtype] : 0;
}

/* nprocs <= 0: omp_get_num_procs(), as the reference does. */
ORACLE_API int oracle_reduce(const void* in, uint64_t n, int dtype, int op, const void* init,
                             void* out, int nprocs) {
  const long P = nprocs > 0 ? nprocs : omp_get_num_procs();
#define BODY(S, T) *(T*)out = reduce_##S((const T*)in, (size_t)n, *(const T*)init, op, P);
  DISPATCH(dtype, BODY)
#undef BODY
  return 0;
}

ORACLE_API int oracle_inclusive_scan(const void* in, void* out, uint64_t n, int dtype, int op) {
#define BODY(S, T) inclusive_scan_##S((const T*)in, (T*)out, (size_t)n, op);
  DISPATCH(dtype, BODY)
#undef BODY
  return 0;
}

ORACLE_API int oracle_exclusive_scan(const void* in, void* out, uint64_t n, int dtype, int op,
                                     const void* init) {
#define BODY(S, T) exclusive_scan_##S((const T*)in, (T*)out, (size_t)n, op, *(const T*)init);
  DISPATCH(dtype, BODY)
#undef BODY
  return 0;
}

static void gather_bytes(const void* src, const size_t* idx, size_t n, size_t bytes, void* dst) {
  long i;
#pragma omp parallel for
  for (i = 0; i < (long)n; i++)
    memcpy((char*)dst + (size_t)i * bytes, (const char*)src + idx[i] * bytes, bytes);
}

/* nthreads <= 0: omp_get_max_threads().  nthreads == 1 is the CPP system. */
ORACLE_API int oracle_sort_keys(void* keys, uint64_t n, int dtype, int descending, int nthreads) {
  const int P = nthreads > 0 ? nthreads : omp_get_max_threads();
#define BODY(S, T) omp_stable_sort_##S((T*)keys, NULL, (size_t)n, descending, P);
  DISPATCH(dtype, BODY)
#undef BODY
  return 0;
}

ORACLE_API int oracle_sort_pairs(void* keys, void* values, uint64_t n, int dtype,
                                 uint64_t value_bytes, int descending, int nthreads) {
  const int P = nthreads > 0 ? nthreads : omp_get_max_threads();
  if (n == 0) return 0;
  size_t* perm = (size_t*)malloc((size_t)n * sizeof(size_t));
  for (size_t i = 0; i < n; i++) perm[i] = i;
#define BODY(S, T) omp_stable_sort_##S((T*)keys, perm, (size_t)n, descending, P);
  DISPATCH(dtype, BODY)
#undef BODY
  void* tmp = malloc((size_t)n * value_bytes);
  memcpy(tmp, values, (size_t)n * value_bytes);
  gather_bytes(tmp, perm, (size_t)n, value_bytes, values);
  free(tmp);
  free(perm);
  return 0;
}

/* stable_sort(_by_key) with a comparator that is not less / greater of a primitive key: the
 * OMP and CPP systems both end in the sequential merge sort for each interval
 * (sequential/sort.inl:103-197 -> stable_merge_sort.inl); any stable sort gives the same
 * result, so the one-interval form is restated.  comparator: 0 operator<, 1 operator>,
 * 2 less_div(param).  values == NULL: keys only. */
ORACLE_API int oracle_comparison_sort(void* keys, void* values, uint64_t n, int dtype, uint64_t value_bytes,
                                      int comparator, long param) {
  if (comparator < 0 || comparator > 2 || (comparator == 2 && param == 0)) return -1;
  if (n == 0) return 0;
  size_t* perm = NULL;
  if (values) {
    perm = (size_t*)malloc((size_t)n * sizeof(size_t));
    for (size_t i = 0; i < n; i++) perm[i] = i;
  }
#define BODY(S, T) comparison_sort_##S((T*)keys, perm, (size_t)n, comparator, param);
  DISPATCH(dtype, BODY)
#undef BODY
  if (values) {
    void* tmp = malloc((size_t)n * value_bytes);
    memcpy(tmp, values, (size_t)n * value_bytes);
    gather_bytes(tmp, perm, (size_t)n, value_bytes, values);
    free(tmp);
    free(perm);
  }
  return 0;
}

/* sequential::merge(_by_key) -- the OMP system inherits it (omp/detail/merge.h:21-22). */
ORACLE_API int oracle_merge_by_key(const void* ka, uint64_t na, const void* kb, uint64_t nb,
                                   const void* va, const void* vb, void* kout, void* vout,
                                   int dtype, uint64_t value_bytes, int descending) {
  const size_t n = (size_t)(na + nb);
  size_t *pa = NULL, *pb = NULL, *po = NULL;
  if (vout) {
    pa = (size_t*)malloc((na ? na : 1) * sizeof(size_t));
    pb = (size_t*)malloc((nb ? nb : 1) * sizeof(size_t));
    po = (size_t*)malloc((n ? n : 1) * sizeof(size_t));
    for (size_t i = 0; i < na; i++) pa[i] = i;
    for (size_t i = 0; i < nb; i++) pb[i] = (size_t)na + i; /* positions in the concatenation */
  }
#define BODY(S, T) \
  seq_merge_##S((const T*)ka, (size_t)na, (const T*)kb, (size_t)nb, (T*)kout, pa, pb, po, descending);
  DISPATCH(dtype, BODY)
#undef BODY
  if (vout) {
    for (size_t i = 0; i < n; i++) {
      const size_t p = po[i];
      const char* src = (p < na) ? (const char*)va + p * value_bytes
                                 : (const char*)vb + (p - (size_t)na) * value_bytes;
      memcpy((char*)vout + i * value_bytes, src, value_bytes);
    }
  }
  free(pa);
  free(pb);
  free(po);
  return 0;
}

ORACLE_API int oracle_merge(const void* a, uint64_t na, const void* b, uint64_t nb, void* out,
                            int dtype, int descending) {
  return oracle_merge_by_key(a, na, b, nb, NULL, NULL, out, NULL, dtype, 0, descending);
}

/* generic::copy_if's core (generic/copy_if.inl:54-93): predicates {0,1} (parallel
 * transform), exclusive scan of them into scatter indices (sequential on OMP),
 * scatter_if (parallel, generic/scatter.inl:73-96); count = last index + last flag.
 * negate != 0 selects the complement (remove_copy_if, generic/remove.inl:112-150). */
static size_t scatter_flagged(const void* in, const unsigned* flags, int negate, size_t n,
                              size_t bytes, void* out) {
  if (n == 0) return 0;
  unsigned* pred = (unsigned*)malloc(n * sizeof(unsigned));
  size_t* idx = (size_t*)malloc(n * sizeof(size_t));
  long i;
#pragma omp parallel for
  for (i = 0; i < (long)n; i++) pred[i] = negate ? !flags[i] : (flags[i] != 0);
  size_t sum = 0;
  for (size_t k = 0; k < n; k++) {
    idx[k] = sum;
    sum += pred[k];
  }
  const size_t count = idx[n - 1] + pred[n - 1];
  if (out != in) {
#pragma omp parallel for
    for (i = 0; i < (long)n; i++)
      if (pred[i]) memcpy((char*)out + idx[i] * bytes, (const char*)in + (size_t)i * bytes, bytes);
  } else {
    /* in-place callers are served from a copy, as the reference's in-place wrappers do
     * (generic/unique.inl:70-74 copies the input to a temporary first) */
    void* tmp = malloc(n * bytes);
    memcpy(tmp, in, n * bytes);
    for (size_t k = 0; k < n; k++)
      if (pred[k]) memcpy((char*)out + idx[k] * bytes, (const char*)tmp + k * bytes, bytes);
    free(tmp);
  }
  free(pred);
  free(idx);
  return count;
}

static int make_pred_flags(const void* tested, size_t n, int dtype, int cmp, const void* thr,
                           unsigned* flags) {
#define BODY(S, T) \
  pred_flags_##S((const T*)tested, n, cmp, thr ? *(const T*)thr : (T)0, flags);
  DISPATCH(dtype, BODY)
#undef BODY
  return 0;
}

/* generic::copy_if with / without stencil (generic/copy_if.inl:97-154). */
ORACLE_API int oracle_copy_if(const void* in, const void* stencil, void* out, uint64_t* num,
                              uint64_t n, uint64_t item_bytes, int stencil_dtype, int cmp,
                              const void* threshold) {
  unsigned* flags = (unsigned*)malloc((n ? n : 1) * sizeof(unsigned));
  if (make_pred_flags(stencil ? stencil : in, (size_t)n, stencil_dtype, cmp, threshold, flags)) {
    free(flags);
    return -1;
  }
  *num = scatter_flagged(in, flags, 0, (size_t)n, (size_t)item_bytes, out);
  free(flags);
  return 0;
}

/* generic::stable_partition_copy (generic/partition.inl:103-119): copy_if into the
 * first output, remove_copy_if into the second. */
ORACLE_API int oracle_partition_copy(const void* in, const void* stencil, void* out_true,
                                     void* out_false, uint64_t* num_true, uint64_t n,
                                     uint64_t item_bytes, int stencil_dtype, int cmp,
                                     const void* threshold) {
  unsigned* flags = (unsigned*)malloc((n ? n : 1) * sizeof(unsigned));
  if (make_pred_flags(stencil ? stencil : in, (size_t)n, stencil_dtype, cmp, threshold, flags)) {
    free(flags);
    return -1;
  }
  *num_true = scatter_flagged(in, flags, 0, (size_t)n, (size_t)item_bytes, out_true);
  scatter_flagged(in, flags, 1, (size_t)n, (size_t)item_bytes, out_false);
  free(flags);
  return 0;
}

/* generic::stable_partition (generic/partition.inl:46-64): copy the range to a
 * temporary, count, remove_copy_if(!pred) to the front, remove_copy_if(pred) behind it. */
ORACLE_API int oracle_stable_partition(void* data, const void* stencil, uint64_t* num_true,
                                       uint64_t n, uint64_t item_bytes, int stencil_dtype, int cmp,
                                       const void* threshold) {
  if (n == 0) {
    *num_true = 0;
    return 0;
  }
  unsigned* flags = (unsigned*)malloc(n * sizeof(unsigned));
  if (make_pred_flags(stencil ? stencil : data, (size_t)n, stencil_dtype, cmp, threshold, flags)) {
    free(flags);
    return -1;
  }
  void* tmp = malloc((size_t)n * item_bytes);
  memcpy(tmp, data, (size_t)n * item_bytes);
  const size_t t = scatter_flagged(tmp, flags, 0, (size_t)n, (size_t)item_bytes, data);
  scatter_flagged(tmp, flags, 1, (size_t)n, (size_t)item_bytes, (char*)data + t * item_bytes);
  *num_true = t;
  free(tmp);
  free(flags);
  return 0;
}

/* generic::unique_copy (generic/unique.inl:59-106) = copy_if with the head flags as
 * stencil; generic::unique_by_key_copy (generic/unique_by_key.inl:56-133) the same on
 * zip(keys, values). */
ORACLE_API int oracle_unique_by_key(const void* keys_in, const void* values_in, void* keys_out,
                                    void* values_out, uint64_t* num, uint64_t n, int key_dtype,
                                    uint64_t value_bytes) {
  unsigned* flags = (unsigned*)malloc((n ? n : 1) * sizeof(unsigned));
#define BODY(S, T) head_flags_##S((const T*)keys_in, (size_t)n, flags);
  DISPATCH(key_dtype, BODY)
#undef BODY
  *num = scatter_flagged(keys_in, flags, 0, (size_t)n, dtype_size(key_dtype), keys_out);
  if (values_out)
    scatter_flagged(values_in, flags, 0, (size_t)n, (size_t)value_bytes, values_out);
  free(flags);
  return 0;
}

ORACLE_API int oracle_unique(const void* in, void* out, uint64_t* num, uint64_t n, int dtype) {
  return oracle_unique_by_key(in, NULL, out, NULL, num, n, dtype, 0);
}

/* generic::reduce_by_key (generic/reduce_by_key.inl:81-136). */
ORACLE_API int oracle_reduce_by_key(const void* keys_in, const void* values_in, void* keys_out,
                                    void* values_out, uint64_t* num_runs, uint64_t n,
                                    int key_dtype, int value_dtype, int op) {
  if (n == 0) {
    *num_runs = 0;
    return 0;
  }
  unsigned* flags = (unsigned*)malloc(n * sizeof(unsigned));
#define BODY(S, T) head_flags_##S((const T*)keys_in, (size_t)n, flags);
  DISPATCH(key_dtype, BODY)
#undef BODY
  const size_t runs =
      scatter_flagged(keys_in, flags, 0, (size_t)n, dtype_size(key_dtype), keys_out);
  size_t runs2 = 0;
#define BODY(S, T) \
  runs2 = reduce_by_flags_##S(flags, (const T*)values_in, (size_t)n, op, (T*)values_out);
  DISPATCH(value_dtype, BODY)
#undef BODY
  free(flags);
  *num_runs = runs;
  return runs == runs2 ? 0 : -2;
}

/* generic::count_if (generic/count.inl:64-74): transform_reduce of pred(x) ? 1 : 0 in the
 * iterator's difference type with plus; the transform is the same 0/1 map copy_if uses. */
ORACLE_API int oracle_count_if(const void* in, uint64_t n, int dtype, int cmp, const void* threshold,
                               uint64_t* count, int nprocs) {
  const long P = nprocs > 0 ? nprocs : omp_get_num_procs();
  unsigned* flags = (unsigned*)malloc((n ? n : 1) * sizeof(unsigned));
#define BODY(S, T) \
  pred_flags_##S((const T*)in, (size_t)n, cmp, threshold ? *(const T*)threshold : (T)0, flags);
  DISPATCH(dtype, BODY)
#undef BODY
  int64_t* ones = (int64_t*)malloc((n ? n : 1) * sizeof(int64_t));
  for (uint64_t i = 0; i < n; i++) ones[i] = flags[i] ? 1 : 0;
  *count = (uint64_t)reduce_i64(ones, (size_t)n, 0, THRUST_AMD_PLUS, P);
  free(ones);
  free(flags);
  return 0;
}

/* Conversion between element types as C++'s static_cast does it (floating point to integer
 * truncates toward zero), the conversion the reference's iterators and function objects
 * apply where an algorithm mixes types: reduce's accumulator has the type of init and
 * every element is converted to it before plus<T> adds (generic/reduce.inl:35-53 with
 * functional.h:211-230), inclusive_scan accumulates in the input's type and converts on
 * output, exclusive_scan accumulates in the type of init (sequential/scan.h:48-115). */
ORACLE_API int oracle_convert(const void* in, int in_dtype, void* out, int out_dtype, uint64_t n) {
#define BODY(S, T) return convert_from_##S((const T*)in, out, out_dtype, (size_t)n);
  DISPATCH(in_dtype, BODY)
#undef BODY
  return -1;
}

/* The four set operations and their by-key forms; values are opaque items of value_bytes
 * that travel with the key the reference's tuple loop emits. */
static int set_operation_impl(int op, const void* ka, uint64_t na, const void* kb, uint64_t nb,
                              const void* va, const void* vb, void* kout, void* vout, uint64_t* num,
                              int dtype, uint64_t value_bytes, int descending) {
  if (op < 0 || op >= THRUST_AMD_SET_OP_COUNT) return -1;
  const size_t cap = (size_t)(na + nb) + 1;
  unsigned char* side = (unsigned char*)malloc(cap);
  size_t* idx = (size_t*)malloc(cap * sizeof(size_t));
  size_t k = 0;
#define BODY(S, T) \
  k = set_operation_##S(op, (const T*)ka, (size_t)na, (const T*)kb, (size_t)nb, descending, side, idx);
  DISPATCH(dtype, BODY)
#undef BODY
  const size_t kbytes = dtype_size(dtype);
  for (size_t o = 0; o < k; o++) {
    const char* ksrc = side[o] ? (const char*)kb : (const char*)ka;
    memcpy((char*)kout + o * kbytes, ksrc + idx[o] * kbytes, kbytes);
    if (vout) {
      const char* vsrc = side[o] ? (const char*)vb : (const char*)va;
      memcpy((char*)vout + o * value_bytes, vsrc + idx[o] * value_bytes, value_bytes);
    }
  }
  free(side);
  free(idx);
  *num = k;
  return 0;
}

ORACLE_API int oracle_set_operation(int op, const void* a, uint64_t na, const void* b, uint64_t nb,
                                    void* out, uint64_t* num, int dtype, int descending) {
  return set_operation_impl(op, a, na, b, nb, NULL, NULL, out, NULL, num, dtype, 0, descending);
}

ORACLE_API int oracle_set_operation_by_key(int op, const void* ka, uint64_t na, const void* kb,
                                           uint64_t nb, const void* va, const void* vb, void* kout,
                                           void* vout, uint64_t* num, int dtype, uint64_t value_bytes,
                                           int descending) {
  return set_operation_impl(op, ka, na, kb, nb, va, vb, kout, vout, num, dtype, value_bytes, descending);
}

/* generic::transform_reduce (generic/transform_reduce.inl:30-48): the system's reduce over
 * the transformed range; generic::transform_inclusive_scan / transform_exclusive_scan
 * (generic/transform_scan.inl:37-97): the system's scans over it. */
ORACLE_API int oracle_transform_reduce(const void* in, uint64_t n, int dtype, int unary, int op,
                                       const void* init, void* out, int nprocs) {
  const long P = nprocs > 0 ? nprocs : omp_get_num_procs();
#define BODY(S, T)                                                     \
  T* f = transformed_##S((const T*)in, (size_t)n, unary);              \
  *(T*)out = reduce_##S(f, (size_t)n, *(const T*)init, op, P);         \
  free(f);
  DISPATCH(dtype, BODY)
#undef BODY
  return 0;
}

ORACLE_API int oracle_transform_inclusive_scan(const void* in, void* out, uint64_t n, int dtype,
                                               int unary, int op) {
#define BODY(S, T)                                            \
  T* f = transformed_##S((const T*)in, (size_t)n, unary);     \
  inclusive_scan_##S(f, (T*)out, (size_t)n, op);              \
  free(f);
  DISPATCH(dtype, BODY)
#undef BODY
  return 0;
}

ORACLE_API int oracle_transform_exclusive_scan(const void* in, void* out, uint64_t n, int dtype,
                                               int unary, int op, const void* init) {
#define BODY(S, T)                                                   \
  T* f = transformed_##S((const T*)in, (size_t)n, unary);            \
  exclusive_scan_##S(f, (T*)out, (size_t)n, op, *(const T*)init);    \
  free(f);
  DISPATCH(dtype, BODY)
#undef BODY
  return 0;
}

ORACLE_API int oracle_inner_product(const void* a, const void* b, uint64_t n, int dtype,
                                    const void* init, void* out, int nprocs) {
  const long P = nprocs > 0 ? nprocs : omp_get_num_procs();
#define BODY(S, T) \
  *(T*)out = inner_product_##S((const T*)a, (const T*)b, (size_t)n, *(const T*)init, P);
  DISPATCH(dtype, BODY)
#undef BODY
  return 0;
}

/* generic::inclusive_scan_by_key / exclusive_scan_by_key with equal_to on the keys
 * (generic/scan_by_key.inl:62-238); head flags as in reduce_by_key. */
ORACLE_API int oracle_inclusive_scan_by_key(const void* keys, const void* values, void* out,
                                            uint64_t n, int key_dtype, int value_dtype, int op) {
  if (n == 0) return 0;
  unsigned* flags = (unsigned*)malloc(n * sizeof(unsigned));
#define BODY(S, T) head_flags_##S((const T*)keys, (size_t)n, flags);
  DISPATCH(key_dtype, BODY)
#undef BODY
#define BODY(S, T) inclusive_scan_by_flags_##S(flags, (const T*)values, (T*)out, (size_t)n, op);
  DISPATCH(value_dtype, BODY)
#undef BODY
  free(flags);
  return 0;
}

ORACLE_API int oracle_exclusive_scan_by_key(const void* keys, const void* values, void* out,
                                            uint64_t n, int key_dtype, int value_dtype, int op,
                                            const void* init) {
  if (n == 0) return 0;
  unsigned* flags = (unsigned*)malloc(n * sizeof(unsigned));
#define BODY(S, T) head_flags_##S((const T*)keys, (size_t)n, flags);
  DISPATCH(key_dtype, BODY)
#undef BODY
#define BODY(S, T) \
  exclusive_scan_by_flags_##S(flags, (const T*)values, (T*)out, (size_t)n, op, *(const T*)init);
  DISPATCH(value_dtype, BODY)
#undef BODY
  free(flags);
  return 0;
}
