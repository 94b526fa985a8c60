/* The drop-in boundary used from plain C (C11, no C++ and no HIP headers): every entry point of
 * include/thrust_amd.h called once on a small input whose answer the reference's own unit
 * tests state (testing/reduce.cu:9-22, scan.cu:24-75, sort.cu:73-104, sort_by_key.cu,
 * reduce_by_key.cu:12-57, unique.cu:60-100, unique_by_key.cu, copy.cu:251-270, partition.cu,
 * merge.cu:11-38, merge_by_key.cu:10-45, set_union.cu / set_intersection.cu / set_difference.cu /
 * set_symmetric_difference.cu "Simple" cases, scan_by_key.cu:10-60, transform_reduce.cu,
 * transform_scan.cu, count.cu, inner_product.cu, sequence.cu:43-76), with the size query and the
 * error returns of the calling convention.  This is the binding a host in another language
 * would write. */
#include <stdint.h>
#include <stdio.h>
#include <string.h>
#include <thrust_amd.h>

static int g_failed = 0, g_checks = 0;
#define CHECK(x)                                                                                     \
  do {                                                                                               \
    int rc_ = (x);                                                                                   \
    ++g_checks;                                                                                      \
    if (rc_) { ++g_failed; printf("FAIL %s:%d %s -> %d (%s)\n", __FILE__, __LINE__, #x, rc_, thrust_amd_error_string(rc_)); } \
  } while (0)
#define EXPECT(c)                                                                   \
  do {                                                                              \
    ++g_checks;                                                                     \
    if (!(c)) { ++g_failed; printf("FAIL %s:%d %s\n", __FILE__, __LINE__, #c); }    \
  } while (0)

/* device copies of host arrays, and back */
static void* to_device(const void* host, size_t bytes) {
  void* d = NULL;
  CHECK(thrust_amd_malloc(&d, bytes ? bytes : 1));
  if (bytes) CHECK(thrust_amd_memcpy(d, host, bytes, THRUST_AMD_H2D, NULL));
  return d;
}
static void* device_buffer(size_t bytes) {
  void* d = NULL;
  CHECK(thrust_amd_malloc(&d, bytes ? bytes : 1));
  return d;
}
static void to_host(void* host, const void* device, size_t bytes) {
  CHECK(thrust_amd_memcpy(host, device, bytes, THRUST_AMD_D2H, NULL));
}
static int same_i32(const int32_t* a, const int32_t* b, size_t n) { return memcmp(a, b, n * sizeof(int32_t)) == 0; }

/* temporary storage the way every entry point asks for it: size query, then the call */
#define WITH_TEMP(call_with)                                   \
  do {                                                         \
    size_t bytes = 0;                                          \
    void* temp = NULL;                                         \
    CHECK(call_with(NULL, &bytes));                            \
    CHECK(thrust_amd_temp_acquire(&temp, bytes, NULL));        \
    CHECK(call_with(temp, &bytes));                            \
    CHECK(thrust_amd_stream_synchronize(NULL));                \
    CHECK(thrust_amd_temp_release(temp, NULL));                \
  } while (0)

int main(void) {
  EXPECT(thrust_amd_version() == THRUST_AMD_VERSION);
  EXPECT(thrust_amd_dtype_size(THRUST_AMD_I8) == 1 && thrust_amd_dtype_size(THRUST_AMD_U16) == 2 &&
         thrust_amd_dtype_size(THRUST_AMD_F32) == 4 && thrust_amd_dtype_size(THRUST_AMD_F64) == 8 &&
         thrust_amd_dtype_size(99) == 0);
  EXPECT(thrust_amd_error_string(0) != NULL && thrust_amd_error_string(1) != NULL);

  uint64_t* d_count = device_buffer(sizeof(uint64_t));
  uint64_t count = 0;

  /* ---- reduce, count_if, inner_product, transform_reduce */
  {
    const int32_t h[3] = {1, -2, 3};
    int32_t out = 0, init = 10;
    void* d = to_device(h, sizeof h);
    void* d_out = device_buffer(sizeof out);
#define CALL(t, b) thrust_amd_reduce(t, b, d, 3, THRUST_AMD_I32, THRUST_AMD_PLUS, &init, d_out, NULL)
    WITH_TEMP(CALL);
#undef CALL
    to_host(&out, d_out, sizeof out);
    EXPECT(out == 12);
    init = 0;
#define CALL(t, b) thrust_amd_reduce(t, b, d, 3, THRUST_AMD_I32, THRUST_AMD_MAX, &init, d_out, NULL)
    WITH_TEMP(CALL);
#undef CALL
    to_host(&out, d_out, sizeof out);
    EXPECT(out == 3);
    /* transform_reduce: sum of the negated elements on top of 10 (testing/transform_reduce.cu:45-58) */
    init = 10;
#define CALL(t, b) thrust_amd_transform_reduce(t, b, d, 3, THRUST_AMD_I32, THRUST_AMD_NEGATE, THRUST_AMD_PLUS, &init, d_out, NULL)
    WITH_TEMP(CALL);
#undef CALL
    to_host(&out, d_out, sizeof out);
    EXPECT(out == 8);
    /* the calling convention: too little temporary storage, an unknown element type */
    size_t small = 0, bytes = 0;
    EXPECT(thrust_amd_reduce(d_out, &small, d, 3, THRUST_AMD_I32, THRUST_AMD_PLUS, &init, d_out, NULL) != 0);
    EXPECT(thrust_amd_reduce(NULL, &bytes, d, 3, 99, THRUST_AMD_PLUS, &init, d_out, NULL) != 0);
    EXPECT(thrust_amd_reduce(NULL, NULL, d, 3, THRUST_AMD_I32, THRUST_AMD_PLUS, &init, d_out, NULL) != 0);
    CHECK(thrust_amd_free(d));
    CHECK(thrust_amd_free(d_out));
  }
  {
    /* testing/count.cu:9-20: [1, 1, 0, 0, 1] holds 0 twice, 1 three times, 2 never */
    const int32_t h[5] = {1, 1, 0, 0, 1};
    void* d = to_device(h, sizeof h);
    for (int32_t value = 0; value < 3; ++value) {
#define CALL(t, b) thrust_amd_count_if(t, b, d, 5, THRUST_AMD_I32, THRUST_AMD_EQ, &value, d_count, NULL)
      WITH_TEMP(CALL);
#undef CALL
      to_host(&count, d_count, sizeof count);
      EXPECT(count == (value == 0 ? 2u : value == 1 ? 3u : 0u));
    }
    CHECK(thrust_amd_free(d));
  }
  {
    /* testing/inner_product.cu:9-22: (1, -2, 3) . (-4, 5, 6) + 3 = 7 */
    const int32_t a[3] = {1, -2, 3}, b[3] = {-4, 5, 6};
    int32_t init = 3, out = 0;
    void *da = to_device(a, sizeof a), *db = to_device(b, sizeof b), *d_out = device_buffer(sizeof out);
#define CALL(t, bb) thrust_amd_inner_product(t, bb, da, db, 3, THRUST_AMD_I32, &init, d_out, NULL)
    WITH_TEMP(CALL);
#undef CALL
    to_host(&out, d_out, sizeof out);
    EXPECT(out == 7);
    CHECK(thrust_amd_free(da)); CHECK(thrust_amd_free(db)); CHECK(thrust_amd_free(d_out));
  }

  /* ---- scans (testing/scan.cu:24-75: input 1 3 -2 4 -5) */
  {
    const int32_t h[5] = {1, 3, -2, 4, -5};
    int32_t got[5], init;
    void *d = to_device(h, sizeof h), *d_out = device_buffer(sizeof h);
#define CALL(t, b) thrust_amd_inclusive_scan(t, b, d, d_out, 5, THRUST_AMD_I32, THRUST_AMD_PLUS, NULL)
    WITH_TEMP(CALL);
#undef CALL
    to_host(got, d_out, sizeof got);
    { const int32_t want[5] = {1, 4, 2, 6, 1}; EXPECT(same_i32(got, want, 5)); }
    CHECK(thrust_amd_inclusive_scan_static(d, d_out, 5, THRUST_AMD_I32, THRUST_AMD_PLUS, NULL));
    CHECK(thrust_amd_stream_synchronize(NULL));
    to_host(got, d_out, sizeof got);
    { const int32_t want[5] = {1, 4, 2, 6, 1}; EXPECT(same_i32(got, want, 5)); }
    init = 3;
#define CALL(t, b) thrust_amd_exclusive_scan(t, b, d, d_out, 5, THRUST_AMD_I32, THRUST_AMD_PLUS, &init, NULL)
    WITH_TEMP(CALL);
#undef CALL
    to_host(got, d_out, sizeof got);
    { const int32_t want[5] = {3, 4, 7, 5, 9}; EXPECT(same_i32(got, want, 5)); }
    /* testing/transform_scan.cu:165-192: negate, then plus */
#define CALL(t, b) thrust_amd_transform_inclusive_scan(t, b, d, d_out, 5, THRUST_AMD_I32, THRUST_AMD_NEGATE, THRUST_AMD_PLUS, NULL)
    WITH_TEMP(CALL);
#undef CALL
    to_host(got, d_out, sizeof got);
    { const int32_t want[5] = {-1, -4, -2, -6, -1}; EXPECT(same_i32(got, want, 5)); }
    init = 3;
#define CALL(t, b) thrust_amd_transform_exclusive_scan(t, b, d, d_out, 5, THRUST_AMD_I32, THRUST_AMD_NEGATE, THRUST_AMD_PLUS, &init, NULL)
    WITH_TEMP(CALL);
#undef CALL
    to_host(got, d_out, sizeof got);
    { const int32_t want[5] = {3, 2, -1, 1, -3}; EXPECT(same_i32(got, want, 5)); }
    CHECK(thrust_amd_free(d)); CHECK(thrust_amd_free(d_out));
  }
  {
    /* testing/scan_by_key.cu:10-60: keys 0 1 1 1 2 3 3, values 1 .. 7 */
    const int32_t k[7] = {0, 1, 1, 1, 2, 3, 3}, v[7] = {1, 2, 3, 4, 5, 6, 7};
    int32_t got[7], init = 10;
    void *dk = to_device(k, sizeof k), *dv = to_device(v, sizeof v), *d_out = device_buffer(sizeof v);
#define CALL(t, b) thrust_amd_inclusive_scan_by_key(t, b, dk, dv, d_out, 7, THRUST_AMD_I32, THRUST_AMD_I32, THRUST_AMD_PLUS, NULL)
    WITH_TEMP(CALL);
#undef CALL
    to_host(got, d_out, sizeof got);
    { const int32_t want[7] = {1, 2, 5, 9, 5, 6, 13}; EXPECT(same_i32(got, want, 7)); }
#define CALL(t, b) thrust_amd_exclusive_scan_by_key(t, b, dk, dv, d_out, 7, THRUST_AMD_I32, THRUST_AMD_I32, THRUST_AMD_PLUS, &init, NULL)
    WITH_TEMP(CALL);
#undef CALL
    to_host(got, d_out, sizeof got);
    { const int32_t want[7] = {10, 10, 12, 15, 10, 10, 16}; EXPECT(same_i32(got, want, 7)); }
    CHECK(thrust_amd_free(dk)); CHECK(thrust_amd_free(dv)); CHECK(thrust_amd_free(d_out));
  }

  /* ---- sorts (testing/sort.cu:73-104, sort_by_key.cu:60-98) */
  {
    const int32_t unsorted_keys[7] = {1, 3, 6, 5, 2, 0, 4}, unsorted_values[7] = {0, 1, 2, 3, 4, 5, 6};
    const int32_t sorted_keys[7] = {0, 1, 2, 3, 4, 5, 6}, sorted_values[7] = {5, 0, 4, 1, 6, 3, 2};
    const int32_t descending_keys[7] = {6, 5, 4, 3, 2, 1, 0};
    int32_t got_k[7], got_v[7];
    void *dk = device_buffer(sizeof unsorted_keys), *dv = device_buffer(sizeof unsorted_values);
    for (int which = 0; which < 4; ++which) {
      CHECK(thrust_amd_memcpy(dk, unsorted_keys, sizeof unsorted_keys, THRUST_AMD_H2D, NULL));
      CHECK(thrust_amd_memcpy(dv, unsorted_values, sizeof unsorted_values, THRUST_AMD_H2D, NULL));
#define RADIX_KEYS(t, b) thrust_amd_sort_keys(t, b, dk, 7, THRUST_AMD_I32, which == 1, 0, 32, NULL)
#define RADIX_PAIRS(t, b) thrust_amd_sort_pairs(t, b, dk, dv, 7, THRUST_AMD_I32, sizeof(int32_t), 0, 0, 32, NULL)
#define MERGE_KEYS(t, b) thrust_amd_merge_sort_keys(t, b, dk, 7, THRUST_AMD_I32, 1, NULL)
#define MERGE_PAIRS(t, b) thrust_amd_merge_sort_pairs(t, b, dk, dv, 7, THRUST_AMD_I32, sizeof(int32_t), 0, NULL)
      if (which == 0 || which == 1) WITH_TEMP(RADIX_KEYS);
      if (which == 2) WITH_TEMP(RADIX_PAIRS);
      if (which == 3) WITH_TEMP(MERGE_PAIRS);
      to_host(got_k, dk, sizeof got_k);
      to_host(got_v, dv, sizeof got_v);
      EXPECT(same_i32(got_k, which == 1 ? descending_keys : sorted_keys, 7));
      if (which >= 2) EXPECT(same_i32(got_v, sorted_values, 7));
    }
    CHECK(thrust_amd_memcpy(dk, unsorted_keys, sizeof unsorted_keys, THRUST_AMD_H2D, NULL));
    WITH_TEMP(MERGE_KEYS);
    to_host(got_k, dk, sizeof got_k);
    EXPECT(same_i32(got_k, descending_keys, 7));
    CHECK(thrust_amd_free(dk)); CHECK(thrust_amd_free(dv));
  }

  /* ---- reduce_by_key, unique, unique_by_key (testing/reduce_by_key.cu:12-57, unique.cu:60-100) */
  {
    const int32_t keys[9] = {11, 11, 21, 20, 21, 21, 21, 37, 37}, values[9] = {0, 1, 2, 3, 4, 5, 6, 7, 8};
    int32_t got_k[9], got_v[9];
    void *dk = to_device(keys, sizeof keys), *dv = to_device(values, sizeof values);
    void *ok = device_buffer(sizeof keys), *ov = device_buffer(sizeof values);
#define CALL(t, b) thrust_amd_reduce_by_key(t, b, dk, dv, ok, ov, d_count, 9, THRUST_AMD_I32, THRUST_AMD_I32, THRUST_AMD_PLUS, NULL)
    WITH_TEMP(CALL);
#undef CALL
    to_host(&count, d_count, sizeof count);
    to_host(got_k, ok, sizeof got_k);
    to_host(got_v, ov, sizeof got_v);
    { const int32_t want_k[5] = {11, 21, 20, 21, 37}, want_v[5] = {1, 2, 3, 15, 15};
      EXPECT(count == 5 && same_i32(got_k, want_k, 5) && same_i32(got_v, want_v, 5)); }
#define CALL(t, b) thrust_amd_unique_by_key(t, b, dk, dv, ok, ov, d_count, 9, THRUST_AMD_I32, sizeof(int32_t), NULL)
    WITH_TEMP(CALL);
#undef CALL
    to_host(&count, d_count, sizeof count);
    to_host(got_k, ok, sizeof got_k);
    to_host(got_v, ov, sizeof got_v);
    { const int32_t want_k[5] = {11, 21, 20, 21, 37}, want_v[5] = {0, 2, 3, 4, 7};
      EXPECT(count == 5 && same_i32(got_k, want_k, 5) && same_i32(got_v, want_v, 5)); }
    CHECK(thrust_amd_free(dk)); CHECK(thrust_amd_free(dv)); CHECK(thrust_amd_free(ok)); CHECK(thrust_amd_free(ov));
  }
  {
    const int32_t h[10] = {11, 11, 12, 20, 29, 21, 21, 31, 31, 37};
    int32_t got[10];
    void *d = to_device(h, sizeof h), *out = device_buffer(sizeof h);
#define CALL(t, b) thrust_amd_unique(t, b, d, out, d_count, 10, THRUST_AMD_I32, NULL)
    WITH_TEMP(CALL);
#undef CALL
    to_host(&count, d_count, sizeof count);
    to_host(got, out, sizeof got);
    { const int32_t want[7] = {11, 12, 20, 29, 21, 31, 37}; EXPECT(count == 7 && same_i32(got, want, 7)); }
    CHECK(thrust_amd_free(d)); CHECK(thrust_amd_free(out));
  }

  /* ---- copy_if, partition_copy, stable_partition (testing/copy.cu:251-270, partition.cu:60-140) */
  {
    const int32_t h[5] = {0, 1, 2, 3, 4}, stencil[5] = {1, 1, 0, 1, 0};
    const int32_t zero = 0;
    int32_t got[5], got_false[5];
    void *d = to_device(h, sizeof h), *ds = to_device(stencil, sizeof stencil);
    void *out = device_buffer(sizeof h), *out_false = device_buffer(sizeof h);
    /* "is true" of the element itself */
#define CALL(t, b) thrust_amd_copy_if(t, b, d, NULL, out, d_count, 5, sizeof(int32_t), THRUST_AMD_I32, THRUST_AMD_NONZERO, NULL, NULL)
    WITH_TEMP(CALL);
#undef CALL
    to_host(&count, d_count, sizeof count);
    to_host(got, out, sizeof got);
    { const int32_t want[4] = {1, 2, 3, 4}; EXPECT(count == 4 && same_i32(got, want, 4)); }
    /* by stencil */
#define CALL(t, b) thrust_amd_copy_if(t, b, d, ds, out, d_count, 5, sizeof(int32_t), THRUST_AMD_I32, THRUST_AMD_NE, &zero, NULL)
    WITH_TEMP(CALL);
#undef CALL
    to_host(&count, d_count, sizeof count);
    to_host(got, out, sizeof got);
    { const int32_t want[3] = {0, 1, 3}; EXPECT(count == 3 && same_i32(got, want, 3)); }
    /* remove_if is the same kernel with the predicate inverted */
#define CALL(t, b) thrust_amd_copy_if(t, b, d, ds, out, d_count, 5, sizeof(int32_t), THRUST_AMD_I32, THRUST_AMD_NE | THRUST_AMD_CMP_NOT, &zero, NULL)
    WITH_TEMP(CALL);
#undef CALL
    to_host(&count, d_count, sizeof count);
    to_host(got, out, sizeof got);
    { const int32_t want[2] = {2, 4}; EXPECT(count == 2 && same_i32(got, want, 2)); }
    /* partition_copy and the in-place partition by "< 2" */
    { const int32_t two = 2;
#define CALL(t, b) thrust_amd_partition_copy(t, b, d, NULL, out, out_false, d_count, 5, sizeof(int32_t), THRUST_AMD_I32, THRUST_AMD_LT, &two, NULL)
      WITH_TEMP(CALL);
#undef CALL
      to_host(&count, d_count, sizeof count);
      to_host(got, out, sizeof got);
      to_host(got_false, out_false, sizeof got_false);
      { const int32_t want_true[2] = {0, 1}, want_false[3] = {2, 3, 4};
        EXPECT(count == 2 && same_i32(got, want_true, 2) && same_i32(got_false, want_false, 3)); }
      { const int32_t mixed[5] = {3, 0, 4, 1, 2};
        CHECK(thrust_amd_memcpy(d, mixed, sizeof mixed, THRUST_AMD_H2D, NULL)); }
#define CALL(t, b) thrust_amd_stable_partition(t, b, d, NULL, d_count, 5, sizeof(int32_t), THRUST_AMD_I32, THRUST_AMD_LT, &two, NULL)
      WITH_TEMP(CALL);
#undef CALL
      to_host(&count, d_count, sizeof count);
      to_host(got, d, sizeof got);
      { const int32_t want[5] = {0, 1, 3, 4, 2}; EXPECT(count == 2 && same_i32(got, want, 5)); }
    }
    CHECK(thrust_amd_free(d)); CHECK(thrust_amd_free(ds)); CHECK(thrust_amd_free(out)); CHECK(thrust_amd_free(out_false));
  }

  /* ---- merge, merge_by_key, the set operations (testing/merge.cu:11-38, merge_by_key.cu:10-45, set_*.cu) */
  {
    const int32_t a[3] = {0, 2, 4}, b[4] = {0, 3, 3, 4}, va[3] = {0, 0, 0}, vb[4] = {1, 1, 1, 1};
    int32_t got_k[7], got_v[7];
    void *da = to_device(a, sizeof a), *db = to_device(b, sizeof b), *dva = to_device(va, sizeof va), *dvb = to_device(vb, sizeof vb);
    void *ok = device_buffer(7 * sizeof(int32_t)), *ov = device_buffer(7 * sizeof(int32_t));
#define CALL(t, bb) thrust_amd_merge(t, bb, da, 3, db, 4, ok, THRUST_AMD_I32, 0, NULL)
    WITH_TEMP(CALL);
#undef CALL
    to_host(got_k, ok, sizeof got_k);
    { const int32_t want[7] = {0, 0, 2, 3, 3, 4, 4}; EXPECT(same_i32(got_k, want, 7)); }
#define CALL(t, bb) thrust_amd_merge_by_key(t, bb, da, 3, db, 4, dva, dvb, ok, ov, THRUST_AMD_I32, sizeof(int32_t), 0, NULL)
    WITH_TEMP(CALL);
#undef CALL
    to_host(got_k, ok, sizeof got_k);
    to_host(got_v, ov, sizeof got_v);
    { const int32_t want_k[7] = {0, 0, 2, 3, 3, 4, 4}, want_v[7] = {0, 1, 0, 1, 1, 0, 1};
      EXPECT(same_i32(got_k, want_k, 7) && same_i32(got_v, want_v, 7)); }
    {
      const int32_t want_union[5] = {0, 2, 3, 3, 4}, want_inter[2] = {0, 4}, want_diff[1] = {2}, want_sym[3] = {2, 3, 3};
      const int32_t* want[4];
      const uint64_t want_n[4] = {1, 2, 3, 5};
      want[THRUST_AMD_SET_DIFFERENCE] = want_diff;
      want[THRUST_AMD_SET_INTERSECTION] = want_inter;
      want[THRUST_AMD_SET_SYMMETRIC_DIFFERENCE] = want_sym;
      want[THRUST_AMD_SET_UNION] = want_union;
      for (int op = 0; op < THRUST_AMD_SET_OP_COUNT; ++op) {
#define CALL(t, bb) thrust_amd_set_operation(t, bb, op, da, 3, db, 4, ok, d_count, THRUST_AMD_I32, 0, NULL)
        WITH_TEMP(CALL);
#undef CALL
        to_host(&count, d_count, sizeof count);
        to_host(got_k, ok, sizeof got_k);
        EXPECT(count == want_n[op] && same_i32(got_k, want[op], (size_t)count));
#define CALL(t, bb) thrust_amd_set_operation_by_key(t, bb, op, da, 3, db, 4, dva, dvb, ok, ov, d_count, THRUST_AMD_I32, sizeof(int32_t), 0, NULL)
        WITH_TEMP(CALL);
#undef CALL
        to_host(&count, d_count, sizeof count);
        to_host(got_k, ok, sizeof got_k);
        to_host(got_v, ov, sizeof got_v);
        EXPECT(count == want_n[op] && same_i32(got_k, want[op], (size_t)count));
        /* values follow their keys: 0 for what came from the first range, 1 from the second */
        if (op == THRUST_AMD_SET_UNION) { const int32_t v[5] = {0, 0, 1, 1, 0}; EXPECT(same_i32(got_v, v, 5)); }
        if (op == THRUST_AMD_SET_SYMMETRIC_DIFFERENCE) { const int32_t v[3] = {0, 1, 1}; EXPECT(same_i32(got_v, v, 3)); }
      }
    }
    CHECK(thrust_amd_free(da)); CHECK(thrust_amd_free(db)); CHECK(thrust_amd_free(dva)); CHECK(thrust_amd_free(dvb));
    CHECK(thrust_amd_free(ok)); CHECK(thrust_amd_free(ov));
  }

  /* ---- fill, sequence, convert, universal memory */
  {
    int32_t got[5];
    float gotf[5];
    const int32_t seven = 7, ten = 10, two = 2;
    void *d = device_buffer(sizeof got), *df = device_buffer(sizeof gotf);
    CHECK(thrust_amd_fill(d, 5, sizeof(int32_t), &seven, NULL));
    to_host(got, d, sizeof got);
    { const int32_t want[5] = {7, 7, 7, 7, 7}; EXPECT(same_i32(got, want, 5)); }
    CHECK(thrust_amd_sequence(d, 5, THRUST_AMD_I32, &ten, &two, NULL));
    to_host(got, d, sizeof got);
    { const int32_t want[5] = {10, 12, 14, 16, 18}; EXPECT(same_i32(got, want, 5)); }
    CHECK(thrust_amd_convert(d, THRUST_AMD_I32, df, THRUST_AMD_F32, 5, NULL));
    to_host(gotf, df, sizeof gotf);
    EXPECT(gotf[0] == 10.0f && gotf[4] == 18.0f);
    CHECK(thrust_amd_free(d)); CHECK(thrust_amd_free(df));
    int32_t* shared = NULL;
    CHECK(thrust_amd_malloc_universal((void**)&shared, 5 * sizeof(int32_t)));
    if (shared) {
      for (int i = 0; i < 5; ++i) shared[i] = 4 - i;  /* plain host stores */
#define CALL(t, b) thrust_amd_sort_keys(t, b, shared, 5, THRUST_AMD_I32, 0, 0, 32, NULL)
      WITH_TEMP(CALL);
#undef CALL
      EXPECT(shared[0] == 0 && shared[4] == 4);     /* plain host loads */
      CHECK(thrust_amd_free_universal(shared));
    }
  }

  /* ---- streams and events, the temporary-storage arena, the launch log */
  {
    void *stream = NULL, *event = NULL, *block = NULL;
    int done = 0;
    int32_t got[4];
    const int32_t h[4] = {4, 3, 2, 1};
    CHECK(thrust_amd_stream_create(&stream));
    CHECK(thrust_amd_event_create(&event));
    void* d = to_device(h, sizeof h);
    CHECK(thrust_amd_profile_enable(1));
    {
      size_t bytes = 0;
      CHECK(thrust_amd_sort_keys(NULL, &bytes, d, 4, THRUST_AMD_I32, 0, 0, 32, stream));
      CHECK(thrust_amd_temp_acquire(&block, bytes, stream));
      CHECK(thrust_amd_sort_keys(block, &bytes, d, 4, THRUST_AMD_I32, 0, 0, 32, stream));
      CHECK(thrust_amd_event_record(event, stream));
      CHECK(thrust_amd_stream_wait_event(NULL, event)); /* the null stream continues after the sort */
      CHECK(thrust_amd_memcpy(got, d, sizeof got, THRUST_AMD_D2H, NULL));
      CHECK(thrust_amd_stream_synchronize(stream));
      CHECK(thrust_amd_stream_query(stream, &done));
      EXPECT(done == 1);
      CHECK(thrust_amd_temp_release(block, stream));
    }
    { const int32_t want[4] = {1, 2, 3, 4}; EXPECT(same_i32(got, want, 4)); }
    EXPECT(thrust_amd_temp_bytes_held() > 0);
    {
      char text[4096];
      size_t needed = 0;
      CHECK(thrust_amd_profile_collect(text, sizeof text, &needed));
      EXPECT(needed > 0 && strstr(text, "sort") != NULL);
      CHECK(thrust_amd_profile_enable(0));
    }
    CHECK(thrust_amd_event_destroy(event));
    CHECK(thrust_amd_stream_destroy(stream));
    CHECK(thrust_amd_free(d));
    CHECK(thrust_amd_temp_trim());
    EXPECT(thrust_amd_temp_bytes_held() == 0);
  }

  CHECK(thrust_amd_free(d_count));
  printf("%d checks, %d failed\n", g_checks, g_failed);
  printf(g_failed ? "FAILED\n" : "PASS c_abi: every entry point from plain C, version %d\n", thrust_amd_version());
  return g_failed ? 1 : 0;
}
