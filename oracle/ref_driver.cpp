// TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.
//
// C bindings around the REAL reference (the Thrust headers under the reference tree),
// compiled twice by oracle/Makefile: once with the OpenMP device system and once with
// the sequential CPP device system.  This file contains no algorithm; it only
// instantiates the reference's templates and gives them the same host-pointer C
// interface as thrust_oracle.c, so that tests can compare the restatement with the
// real thing and write golden vectors, and the benchmark can time the reference's
// OMP path as CPU baseline.  Built only into oracle/_ref/, which is not committed.
//
// The same file also compiles against any other implementation of the same API: with
// -DDRIVER_POLICY=thrust::host -DDRIVER_HOST_POINTERS every call below runs on the host
// system of whichever <thrust/...> headers are first on the include path, over raw
// pointers.  The tests build it that way against this repository's own headers to compare
// their host system with the reference's, call for call.
#include <thrust/copy.h>
#include <thrust/count.h>
#include <thrust/device_ptr.h>
#include <thrust/execution_policy.h>
#include <thrust/functional.h>
#include <thrust/inner_product.h>
#include <thrust/merge.h>
#include <thrust/partition.h>
#include <thrust/reduce.h>
#include <thrust/scan.h>
#include <thrust/random.h>
#include <thrust/set_operations.h>
#include <thrust/shuffle.h>
#include <thrust/sort.h>
#include <thrust/transform_reduce.h>
#include <thrust/transform_scan.h>
#include <thrust/unique.h>

#include <cstdint>
#include <cstring>

#include "../include/thrust_amd.h"

#define REF_API extern "C" __attribute__((visibility("default")))

namespace {

#ifndef DRIVER_POLICY
#define DRIVER_POLICY thrust::device
#endif
#ifdef DRIVER_HOST_POINTERS
template <typename T> T* dp(void* p) { return (T*)p; }
template <typename T> const T* dp(const void* p) { return (const T*)p; }
#else
template <typename T> thrust::device_ptr<T> dp(void* p) { return thrust::device_pointer_cast((T*)p); }
template <typename T> thrust::device_ptr<const T> dp(const void* p) { return thrust::device_pointer_cast((const T*)p); }
#endif

template <typename F>
int with_dtype(int dtype, F&& f) {
  switch (dtype) {
    case THRUST_AMD_I8: return f((int8_t)0);
    case THRUST_AMD_U8: return f((uint8_t)0);
    case THRUST_AMD_I16: return f((int16_t)0);
    case THRUST_AMD_U16: return f((uint16_t)0);
    case THRUST_AMD_I32: return f((int32_t)0);
    case THRUST_AMD_U32: return f((uint32_t)0);
    case THRUST_AMD_I64: return f((int64_t)0);
    case THRUST_AMD_U64: return f((uint64_t)0);
    case THRUST_AMD_F32: return f((float)0);
    case THRUST_AMD_F64: return f((double)0);
    default: return -1;
  }
}

template <typename F>
int with_bytes(uint64_t bytes, F&& f) {
  switch (bytes) {
    case 1: return f((uint8_t)0);
    case 2: return f((uint16_t)0);
    case 4: return f((uint32_t)0);
    case 8: return f((uint64_t)0);
    default: return -1;
  }
}

template <typename T, typename F>
int with_op(int op, F&& f) {
  switch (op) {
    case THRUST_AMD_PLUS: return f(thrust::plus<T>());
    case THRUST_AMD_MIN: return f(thrust::minimum<T>());
    case THRUST_AMD_MAX: return f(thrust::maximum<T>());
    default: return -1;
  }
}

template <typename T>
struct cmp_pred {
  int cmp;
  T t;
  __host__ __device__ bool operator()(const T& x) const {
    switch (cmp) {
      case THRUST_AMD_LT: return x < t;
      case THRUST_AMD_LE: return x <= t;
      case THRUST_AMD_GT: return x > t;
      case THRUST_AMD_GE: return x >= t;
      case THRUST_AMD_EQ: return x == t;
      case THRUST_AMD_NE: return x != t;
      default: return x != T(0);
    }
  }
};

template <typename T>
cmp_pred<T> make_pred(int cmp, const void* thr) {
  cmp_pred<T> p;
  p.cmp = cmp;
  p.t = thr ? *(const T*)thr : T(0);
  return p;
}

}  // namespace

// 1 = OMP device system, 0 = CPP
#if defined(THRUST_DEVICE_SYSTEM) && defined(THRUST_DEVICE_SYSTEM_OMP) && !defined(DRIVER_HOST_POINTERS)
REF_API int ref_is_omp(void) { return THRUST_DEVICE_SYSTEM == THRUST_DEVICE_SYSTEM_OMP; }
#else
REF_API int ref_is_omp(void) { return 0; }
#endif

REF_API int ref_reduce(const void* in, uint64_t n, int dtype, int op, const void* init, void* out) {
  return with_dtype(dtype, [&](auto z) {
    using T = decltype(z);
    return with_op<T>(op, [&](auto o) {
      *(T*)out = thrust::reduce(DRIVER_POLICY, dp<T>(in), dp<T>(in) + n, *(const T*)init, o);
      return 0;
    });
  });
}

REF_API int ref_inclusive_scan(const void* in, void* out, uint64_t n, int dtype, int op) {
  return with_dtype(dtype, [&](auto z) {
    using T = decltype(z);
    return with_op<T>(op, [&](auto o) {
      thrust::inclusive_scan(DRIVER_POLICY, dp<T>(in), dp<T>(in) + n, dp<T>(out), o);
      return 0;
    });
  });
}

REF_API int ref_exclusive_scan(const void* in, void* out, uint64_t n, int dtype, int op,
                               const void* init) {
  return with_dtype(dtype, [&](auto z) {
    using T = decltype(z);
    return with_op<T>(op, [&](auto o) {
      thrust::exclusive_scan(DRIVER_POLICY, dp<T>(in), dp<T>(in) + n, dp<T>(out), *(const T*)init, o);
      return 0;
    });
  });
}

REF_API int ref_sort_keys(void* keys, uint64_t n, int dtype, int descending) {
  return with_dtype(dtype, [&](auto z) {
    using T = decltype(z);
    if (descending) thrust::sort(DRIVER_POLICY, dp<T>(keys), dp<T>(keys) + n, thrust::greater<T>());
    else thrust::sort(DRIVER_POLICY, dp<T>(keys), dp<T>(keys) + n);
    return 0;
  });
}

REF_API int ref_sort_pairs(void* keys, void* values, uint64_t n, int dtype, uint64_t value_bytes,
                           int descending) {
  return with_dtype(dtype, [&](auto z) {
    using T = decltype(z);
    return with_bytes(value_bytes, [&](auto vz) {
      using V = decltype(vz);
      if (descending)
        thrust::stable_sort_by_key(DRIVER_POLICY, dp<T>(keys), dp<T>(keys) + n, dp<V>(values), thrust::greater<T>());
      else
        thrust::stable_sort_by_key(DRIVER_POLICY, dp<T>(keys), dp<T>(keys) + n, dp<V>(values));
      return 0;
    });
  });
}

namespace {
// User-defined comparators: not thrust::less / thrust::greater, so the reference takes its
// comparison sort (sequential/sort.inl:103-197 via the OMP system's intervals).
template <typename T> struct user_less {
  __host__ __device__ bool operator()(const T& a, const T& b) const { return a < b; }
};
template <typename T> struct user_greater {
  __host__ __device__ bool operator()(const T& a, const T& b) const { return b < a; }
};
template <typename T> struct user_less_div {  // testing/stable_sort.cu:43-47 with a parameter
  int d;
  __host__ __device__ bool operator()(const T& a, const T& b) const { return ((int)a) / d < ((int)b) / d; }
};
template <typename T, typename C>
void comparison_sort(void* keys, void* values, uint64_t n, uint64_t value_bytes, C comp) {
  if (!values) {
    thrust::stable_sort(DRIVER_POLICY, dp<T>(keys), dp<T>(keys) + n, comp);
    return;
  }
  with_bytes(value_bytes, [&](auto vz) {
    using V = decltype(vz);
    thrust::stable_sort_by_key(DRIVER_POLICY, dp<T>(keys), dp<T>(keys) + n, dp<V>(values), comp);
    return 0;
  });
}
}  // namespace

REF_API int ref_comparison_sort(void* keys, void* values, uint64_t n, int dtype, uint64_t value_bytes,
                                int comparator, long param) {
  return with_dtype(dtype, [&](auto z) {
    using T = decltype(z);
    if (comparator == 0) comparison_sort<T>(keys, values, n, value_bytes, user_less<T>());
    else if (comparator == 1) comparison_sort<T>(keys, values, n, value_bytes, user_greater<T>());
    else if (comparator == 2 && param != 0) comparison_sort<T>(keys, values, n, value_bytes, user_less_div<T>{(int)param});
    else return -1;
    return 0;
  });
}

REF_API int ref_merge(const void* a, uint64_t na, const void* b, uint64_t nb, void* out, int dtype,
                      int descending) {
  return with_dtype(dtype, [&](auto z) {
    using T = decltype(z);
    if (descending)
      thrust::merge(DRIVER_POLICY, dp<T>(a), dp<T>(a) + na, dp<T>(b), dp<T>(b) + nb, dp<T>(out), thrust::greater<T>());
    else
      thrust::merge(DRIVER_POLICY, dp<T>(a), dp<T>(a) + na, dp<T>(b), dp<T>(b) + nb, dp<T>(out));
    return 0;
  });
}

REF_API int ref_merge_by_key(const void* ka, uint64_t na, const void* kb, uint64_t nb,
                             const void* va, const void* vb, void* kout, void* vout, int dtype,
                             uint64_t value_bytes, int descending) {
  return with_dtype(dtype, [&](auto z) {
    using T = decltype(z);
    return with_bytes(value_bytes, [&](auto vz) {
      using V = decltype(vz);
      if (descending)
        thrust::merge_by_key(DRIVER_POLICY, dp<T>(ka), dp<T>(ka) + na, dp<T>(kb), dp<T>(kb) + nb,
                             dp<V>(va), dp<V>(vb), dp<T>(kout), dp<V>(vout), thrust::greater<T>());
      else
        thrust::merge_by_key(DRIVER_POLICY, dp<T>(ka), dp<T>(ka) + na, dp<T>(kb), dp<T>(kb) + nb,
                             dp<V>(va), dp<V>(vb), dp<T>(kout), dp<V>(vout));
      return 0;
    });
  });
}

REF_API int ref_copy_if(const void* in, const void* stencil, void* out, uint64_t* num, uint64_t n,
                        uint64_t item_bytes, int stencil_dtype, int cmp, const void* threshold) {
  return with_dtype(stencil_dtype, [&](auto z) {
    using T = decltype(z);
    const cmp_pred<T> pred = make_pred<T>(cmp, threshold);
    if (!stencil) {
      *num = thrust::copy_if(DRIVER_POLICY, dp<T>(in), dp<T>(in) + n, dp<T>(out), pred) - dp<T>(out);
      return 0;
    }
    return with_bytes(item_bytes, [&](auto vz) {
      using V = decltype(vz);
      *num = thrust::copy_if(DRIVER_POLICY, dp<V>(in), dp<V>(in) + n, dp<T>(stencil), dp<V>(out), pred) - dp<V>(out);
      return 0;
    });
  });
}

REF_API int ref_partition_copy(const void* in, const void* stencil, void* out_true, void* out_false,
                               uint64_t* num_true, uint64_t n, uint64_t item_bytes,
                               int stencil_dtype, int cmp, const void* threshold) {
  return with_dtype(stencil_dtype, [&](auto z) {
    using T = decltype(z);
    const cmp_pred<T> pred = make_pred<T>(cmp, threshold);
    if (!stencil) {
      *num_true = thrust::stable_partition_copy(DRIVER_POLICY, dp<T>(in), dp<T>(in) + n,
                                                dp<T>(out_true), dp<T>(out_false), pred).first - dp<T>(out_true);
      return 0;
    }
    return with_bytes(item_bytes, [&](auto vz) {
      using V = decltype(vz);
      *num_true = thrust::stable_partition_copy(DRIVER_POLICY, dp<V>(in), dp<V>(in) + n, dp<T>(stencil),
                                                dp<V>(out_true), dp<V>(out_false), pred).first - dp<V>(out_true);
      return 0;
    });
  });
}

REF_API int ref_stable_partition(void* data, const void* stencil, uint64_t* num_true, uint64_t n,
                                 uint64_t item_bytes, int stencil_dtype, int cmp,
                                 const void* threshold) {
  return with_dtype(stencil_dtype, [&](auto z) {
    using T = decltype(z);
    const cmp_pred<T> pred = make_pred<T>(cmp, threshold);
    if (!stencil) {
      *num_true = thrust::stable_partition(DRIVER_POLICY, dp<T>(data), dp<T>(data) + n, pred) - dp<T>(data);
      return 0;
    }
    return with_bytes(item_bytes, [&](auto vz) {
      using V = decltype(vz);
      *num_true = thrust::stable_partition(DRIVER_POLICY, dp<V>(data), dp<V>(data) + n, dp<T>(stencil), pred) - dp<V>(data);
      return 0;
    });
  });
}

REF_API int ref_unique(const void* in, void* out, uint64_t* num, uint64_t n, int dtype) {
  return with_dtype(dtype, [&](auto z) {
    using T = decltype(z);
    if (in == out) *num = thrust::unique(DRIVER_POLICY, dp<T>(out), dp<T>(out) + n) - dp<T>(out);
    else *num = thrust::unique_copy(DRIVER_POLICY, dp<T>(in), dp<T>(in) + n, dp<T>(out)) - dp<T>(out);
    return 0;
  });
}

REF_API int ref_unique_by_key(const void* keys_in, const void* values_in, void* keys_out,
                              void* values_out, uint64_t* num, uint64_t n, int key_dtype,
                              uint64_t value_bytes) {
  return with_dtype(key_dtype, [&](auto z) {
    using T = decltype(z);
    return with_bytes(value_bytes, [&](auto vz) {
      using V = decltype(vz);
      if (keys_in == keys_out)
        *num = thrust::unique_by_key(DRIVER_POLICY, dp<T>(keys_out), dp<T>(keys_out) + n, dp<V>(values_out)).first - dp<T>(keys_out);
      else
        *num = thrust::unique_by_key_copy(DRIVER_POLICY, dp<T>(keys_in), dp<T>(keys_in) + n, dp<V>(values_in),
                                          dp<T>(keys_out), dp<V>(values_out)).first - dp<T>(keys_out);
      return 0;
    });
  });
}

// Value types are limited to the ones the library's tests and configs use, to keep the
// compile time of the reference's zip-iterator scan in bounds.
REF_API int ref_reduce_by_key(const void* keys_in, const void* values_in, void* keys_out,
                              void* values_out, uint64_t* num_runs, uint64_t n, int key_dtype,
                              int value_dtype, int op) {
  auto run = [&](auto kz, auto vz) {
    using K = decltype(kz);
    using V = decltype(vz);
    return with_op<V>(op, [&](auto o) {
      *num_runs = thrust::reduce_by_key(DRIVER_POLICY, dp<K>(keys_in), dp<K>(keys_in) + n, dp<V>(values_in),
                                        dp<K>(keys_out), dp<V>(values_out), thrust::equal_to<K>(), o).first - dp<K>(keys_out);
      return 0;
    });
  };
  auto by_value = [&](auto kz) {
    switch (value_dtype) {
      case THRUST_AMD_I32: return run(kz, (int32_t)0);
      case THRUST_AMD_I64: return run(kz, (int64_t)0);
      case THRUST_AMD_F32: return run(kz, (float)0);
      case THRUST_AMD_F64: return run(kz, (double)0);
      default: return -1;
    }
  };
  switch (key_dtype) {
    case THRUST_AMD_I32: return by_value((int32_t)0);
    case THRUST_AMD_U32: return by_value((uint32_t)0);
    case THRUST_AMD_I64: return by_value((int64_t)0);
    case THRUST_AMD_U64: return by_value((uint64_t)0);
    case THRUST_AMD_F32: return by_value((float)0);
    default: return -1;
  }
}

REF_API int ref_count_if(const void* in, uint64_t n, int dtype, int cmp, const void* threshold,
                         uint64_t* count) {
  return with_dtype(dtype, [&](auto z) {
    using T = decltype(z);
    *count = (uint64_t)thrust::count_if(DRIVER_POLICY, dp<T>(in), dp<T>(in) + n, make_pred<T>(cmp, threshold));
    return 0;
  });
}

REF_API int ref_inner_product(const void* a, const void* b, uint64_t n, int dtype, const void* init,
                              void* out) {
  return with_dtype(dtype, [&](auto z) {
    using T = decltype(z);
    *(T*)out = thrust::inner_product(DRIVER_POLICY, dp<T>(a), dp<T>(a) + n, dp<T>(b), *(const T*)init);
    return 0;
  });
}

// Mixed element types through the real reference, for the pairs the tests use: x is int32
// or float32, the other type is the other one of the two.
REF_API int ref_convert(const void* in, int in_dtype, void* out, int out_dtype, uint64_t n) {
  return with_dtype(in_dtype, [&](auto zi) {
    using TI = decltype(zi);
    return with_dtype(out_dtype, [&](auto zo) {
      using TO = decltype(zo);
      thrust::copy(DRIVER_POLICY, dp<TI>(in), dp<TI>(in) + n, dp<TO>(out));  // converting copy
      return 0;
    });
  });
}
REF_API int ref_reduce_mixed(const void* in, int in_dtype, uint64_t n, int init_dtype, const void* init, void* out) {
  if (in_dtype == THRUST_AMD_F32 && init_dtype == THRUST_AMD_I32)
    *(int32_t*)out = thrust::reduce(DRIVER_POLICY, dp<float>(in), dp<float>(in) + n, *(const int32_t*)init);
  else if (in_dtype == THRUST_AMD_I32 && init_dtype == THRUST_AMD_F32)
    *(float*)out = thrust::reduce(DRIVER_POLICY, dp<int32_t>(in), dp<int32_t>(in) + n, *(const float*)init);
  else
    return -1;
  return 0;
}
// inclusive_scan(in, out) and exclusive_scan(in, out, init) with out of the other type;
// init has init_dtype (THRUST_AMD_I32 or THRUST_AMD_F32); exclusive < 0: inclusive scan
REF_API int ref_scan_mixed(const void* in, int in_dtype, void* out, uint64_t n, int exclusive, int init_dtype,
                           const void* init) {
  auto run = [&](auto zi, auto zo) {
    using TI = decltype(zi);
    using TO = decltype(zo);
    if (exclusive < 0) thrust::inclusive_scan(DRIVER_POLICY, dp<TI>(in), dp<TI>(in) + n, dp<TO>(out));
    else if (init_dtype == THRUST_AMD_I32)
      thrust::exclusive_scan(DRIVER_POLICY, dp<TI>(in), dp<TI>(in) + n, dp<TO>(out), *(const int32_t*)init);
    else
      thrust::exclusive_scan(DRIVER_POLICY, dp<TI>(in), dp<TI>(in) + n, dp<TO>(out), *(const float*)init);
    return 0;
  };
  if (in_dtype == THRUST_AMD_F32) return run((float)0, (int32_t)0);
  if (in_dtype == THRUST_AMD_I32) return run((int32_t)0, (float)0);
  return -1;
}

namespace {
// The real set operations; C is thrust::less<K> or thrust::greater<K>.
template <typename K, typename C>
uint64_t run_set_operation(int op, const void* a, uint64_t na, const void* b, uint64_t nb, void* out, C comp) {
  auto a0 = dp<K>(a), b0 = dp<K>(b);
  auto o0 = dp<K>(out);
  switch (op) {
    case THRUST_AMD_SET_DIFFERENCE: return thrust::set_difference(DRIVER_POLICY, a0, a0 + na, b0, b0 + nb, o0, comp) - o0;
    case THRUST_AMD_SET_INTERSECTION: return thrust::set_intersection(DRIVER_POLICY, a0, a0 + na, b0, b0 + nb, o0, comp) - o0;
    case THRUST_AMD_SET_SYMMETRIC_DIFFERENCE:
      return thrust::set_symmetric_difference(DRIVER_POLICY, a0, a0 + na, b0, b0 + nb, o0, comp) - o0;
    default: return thrust::set_union(DRIVER_POLICY, a0, a0 + na, b0, b0 + nb, o0, comp) - o0;
  }
}
template <typename K, typename V, typename C>
uint64_t run_set_operation_by_key(int op, const void* ka, uint64_t na, const void* kb, uint64_t nb, const void* va,
                                  const void* vb, void* kout, void* vout, C comp) {
  auto a0 = dp<K>(ka), b0 = dp<K>(kb);
  auto v1 = dp<V>(va), v2 = dp<V>(vb);
  auto ko = dp<K>(kout);
  auto vo = dp<V>(vout);
  switch (op) {
    case THRUST_AMD_SET_DIFFERENCE:
      return thrust::set_difference_by_key(DRIVER_POLICY, a0, a0 + na, b0, b0 + nb, v1, v2, ko, vo, comp).first - ko;
    case THRUST_AMD_SET_INTERSECTION:
      return thrust::set_intersection_by_key(DRIVER_POLICY, a0, a0 + na, b0, b0 + nb, v1, ko, vo, comp).first - ko;
    case THRUST_AMD_SET_SYMMETRIC_DIFFERENCE:
      return thrust::set_symmetric_difference_by_key(DRIVER_POLICY, a0, a0 + na, b0, b0 + nb, v1, v2, ko, vo, comp).first - ko;
    default: return thrust::set_union_by_key(DRIVER_POLICY, a0, a0 + na, b0, b0 + nb, v1, v2, ko, vo, comp).first - ko;
  }
}
}  // namespace

REF_API int ref_set_operation(int op, const void* a, uint64_t na, const void* b, uint64_t nb, void* out,
                              uint64_t* num, int dtype, int descending) {
  return with_dtype(dtype, [&](auto z) {
    using K = decltype(z);
    *num = descending ? run_set_operation<K>(op, a, na, b, nb, out, thrust::greater<K>())
                      : run_set_operation<K>(op, a, na, b, nb, out, thrust::less<K>());
    return 0;
  });
}

// Keys of the types the fixtures use; values as opaque 4- or 8-byte items.
REF_API int ref_set_operation_by_key(int op, const void* ka, uint64_t na, const void* kb, uint64_t nb,
                                     const void* va, const void* vb, void* kout, void* vout, uint64_t* num,
                                     int dtype, uint64_t value_bytes, int descending) {
  auto run = [&](auto kz, auto vz) {
    using K = decltype(kz);
    using V = decltype(vz);
    *num = descending ? run_set_operation_by_key<K, V>(op, ka, na, kb, nb, va, vb, kout, vout, thrust::greater<K>())
                      : run_set_operation_by_key<K, V>(op, ka, na, kb, nb, va, vb, kout, vout, thrust::less<K>());
    return 0;
  };
  auto by_value = [&](auto kz) {
    switch (value_bytes) {
      case 4: return run(kz, (uint32_t)0);
      case 8: return run(kz, (uint64_t)0);
      default: return -1;
    }
  };
  switch (dtype) {
    case THRUST_AMD_I32: return by_value((int32_t)0);
    case THRUST_AMD_U32: return by_value((uint32_t)0);
    case THRUST_AMD_U64: return by_value((uint64_t)0);
    case THRUST_AMD_F32: return by_value((float)0);
    default: return -1;
  }
}

namespace {
template <typename T, typename F>
int with_unary(int unary, F&& f) {
  switch (unary) {
    case THRUST_AMD_IDENTITY: return f(thrust::identity<T>());
    case THRUST_AMD_NEGATE: return f(thrust::negate<T>());
    case THRUST_AMD_SQUARE: return f(thrust::square<T>());
    default: return -1;
  }
}
}  // namespace

REF_API int ref_transform_reduce(const void* in, uint64_t n, int dtype, int unary, int op,
                                 const void* init, void* out) {
  return with_dtype(dtype, [&](auto z) {
    using T = decltype(z);
    return with_unary<T>(unary, [&](auto u) {
      return with_op<T>(op, [&](auto o) {
        *(T*)out = thrust::transform_reduce(DRIVER_POLICY, dp<T>(in), dp<T>(in) + n, u, *(const T*)init, o);
        return 0;
      });
    });
  });
}

REF_API int ref_transform_inclusive_scan(const void* in, void* out, uint64_t n, int dtype, int unary,
                                         int op) {
  return with_dtype(dtype, [&](auto z) {
    using T = decltype(z);
    return with_unary<T>(unary, [&](auto u) {
      return with_op<T>(op, [&](auto o) {
        thrust::transform_inclusive_scan(DRIVER_POLICY, dp<T>(in), dp<T>(in) + n, dp<T>(out), u, o);
        return 0;
      });
    });
  });
}

REF_API int ref_transform_exclusive_scan(const void* in, void* out, uint64_t n, int dtype, int unary,
                                         int op, const void* init) {
  return with_dtype(dtype, [&](auto z) {
    using T = decltype(z);
    return with_unary<T>(unary, [&](auto u) {
      return with_op<T>(op, [&](auto o) {
        thrust::transform_exclusive_scan(DRIVER_POLICY, dp<T>(in), dp<T>(in) + n, dp<T>(out), u, *(const T*)init, o);
        return 0;
      });
    });
  });
}

namespace {
template <typename F>
int with_key_value(int key_dtype, int value_dtype, F&& run) {
  auto by_value = [&](auto kz) {
    switch (value_dtype) {
      case THRUST_AMD_I32: return run(kz, (int32_t)0);
      case THRUST_AMD_I64: return run(kz, (int64_t)0);
      case THRUST_AMD_F32: return run(kz, (float)0);
      case THRUST_AMD_F64: return run(kz, (double)0);
      default: return -1;
    }
  };
  switch (key_dtype) {
    case THRUST_AMD_I32: return by_value((int32_t)0);
    case THRUST_AMD_U32: return by_value((uint32_t)0);
    case THRUST_AMD_I64: return by_value((int64_t)0);
    case THRUST_AMD_U64: return by_value((uint64_t)0);
    case THRUST_AMD_F32: return by_value((float)0);
    default: return -1;
  }
}
}  // namespace

REF_API int ref_inclusive_scan_by_key(const void* keys, const void* values, void* out, uint64_t n,
                                      int key_dtype, int value_dtype, int op) {
  return with_key_value(key_dtype, value_dtype, [&](auto kz, auto vz) {
    using K = decltype(kz);
    using V = decltype(vz);
    return with_op<V>(op, [&](auto o) {
      thrust::inclusive_scan_by_key(DRIVER_POLICY, dp<K>(keys), dp<K>(keys) + n, dp<V>(values), dp<V>(out),
                                    thrust::equal_to<K>(), o);
      return 0;
    });
  });
}

REF_API int ref_exclusive_scan_by_key(const void* keys, const void* values, void* out, uint64_t n,
                                      int key_dtype, int value_dtype, int op, const void* init) {
  return with_key_value(key_dtype, value_dtype, [&](auto kz, auto vz) {
    using K = decltype(kz);
    using V = decltype(vz);
    return with_op<V>(op, [&](auto o) {
      thrust::exclusive_scan_by_key(DRIVER_POLICY, dp<K>(keys), dp<K>(keys) + n, dp<V>(values), dp<V>(out),
                                    *(const V*)init, thrust::equal_to<K>(), o);
      return 0;
    });
  });
}

// thrust::shuffle_copy with thrust::default_random_engine(seed): the permutation the library
// draws for that generator (in and out may not overlap).
REF_API int ref_shuffle_copy(const void* in, void* out, uint64_t n, int dtype, uint32_t seed) {
  return with_dtype(dtype, [&](auto z) {
    using T = decltype(z);
    thrust::default_random_engine g(seed);
    thrust::shuffle_copy(DRIVER_POLICY, dp<T>(in), dp<T>(in) + n, dp<T>(out), g);
    return 0;
  });
}
// thrust::shuffle in place, same generator.
REF_API int ref_shuffle(void* data, uint64_t n, int dtype, uint32_t seed) {
  return with_dtype(dtype, [&](auto z) {
    using T = decltype(z);
    thrust::default_random_engine g(seed);
    thrust::shuffle(DRIVER_POLICY, dp<T>(data), dp<T>(data) + n, g);
    return 0;
  });
}

