"""The seeded cases of the golden fixtures: one function per benchmark configuration, returning
{name: output array} when run on an implementation with the Oracle/Reference interface
(oracle.cpu) or on the device (tests pass an adapter).  Shared by the fixture writer
(which runs the REAL reference) and by the tests (which run the restatement / the GPU)."""
import hashlib

import numpy as np

from thrust_amd import datagen

LT = 0
SMALL = {"c1": 1 << 14, "c2": 1 << 14, "c3": 1 << 13, "c4": 1 << 15, "c5": 1 << 14, "c6": 1 << 15, "c7": 1 << 14,
         "c8": 1 << 14}
LARGE = {"c1": 1 << 22, "c2": 1 << 22, "c3": 1 << 21, "c4": 1 << 22, "c5": 1 << 22, "c6": 1 << 22, "c7": 1 << 22,
         "c8": 1 << 21}


def c1(impl, n):
    x = datagen.c1_int32(n)
    x64 = x.astype(np.int64) * 1000003
    return {
        "c1.reduce_i32": np.array([impl.reduce(x)], np.int32),
        "c1.reduce_i32_init7": np.array([impl.reduce(x, init=7)], np.int32),
        "c1.inclusive_scan_i32": impl.inclusive_scan(x),
        "c1.exclusive_scan_i32_init5": impl.exclusive_scan(x, 5),
        "c1.reduce_i64": np.array([impl.reduce(x64)], np.int64),
        "c1.inclusive_scan_i64": impl.inclusive_scan(x64),
    }


def c2(impl, n):
    # impl must be the sequential (CPP) system for the float case: the multi-thread OMP
    # layout of +-0.0 depends on the thread count
    k = datagen.c2_uint32(n)
    f = datagen.c2_float32(n)
    return {
        "c2.sort_u32": impl.sort_keys(k),
        "c2.sort_u32_desc": impl.sort_keys(k, descending=True),
        "c2.sort_f32_bits": impl.sort_keys(f).view(np.uint32),
        "c2.sort_i32": impl.sort_keys(k.view(np.int32)),
    }


def c3(impl, n):
    out = {}
    v = np.arange(n, dtype=np.uint32)
    for kind in ("full", "low16", "skew90"):
        k = datagen.c3_uint64(n, kind)
        ko, vo = impl.sort_pairs(k, v)
        out[f"c3.{kind}.keys"] = ko
        out[f"c3.{kind}.values"] = vo
    return out


def c4(impl, n, float_sums=True):
    out = {}
    for mean in (8, 1000):
        k, v = datagen.c4_segments(n, mean)
        ko, vo = impl.reduce_by_key(k, v)
        out[f"c4.m{mean}.rbk_keys"] = ko
        if float_sums:
            out[f"c4.m{mean}.rbk_sums_f32"] = vo
        iv = (v * 1000).astype(np.int32)
        _, io = impl.reduce_by_key(k, iv)
        out[f"c4.m{mean}.rbk_sums_i32"] = io
        uk, uv = impl.unique_by_key(k, v)
        out[f"c4.m{mean}.ubk_keys"] = uk
        out[f"c4.m{mean}.ubk_values_bits"] = uv.view(np.uint32)
    return out


def c5(impl, n):
    out = {}
    x = datagen.c5_float32(n)
    for t in (0.5, 0.05):
        out[f"c5.copy_if_lt{t}"] = impl.copy_if(x, LT, t).view(np.uint32)
        part, split = impl.stable_partition(x, LT, t)
        out[f"c5.stable_partition_lt{t}"] = part.view(np.uint32)
        out[f"c5.stable_partition_lt{t}.split"] = np.array([split], np.uint64)
    (ka, va), (kb, vb) = datagen.c5_merge_inputs(n // 2)
    ko, vo = impl.merge_by_key(ka, kb, va, vb)
    out["c5.merge_keys"] = ko
    out["c5.merge_values"] = vo
    return out


def c6(impl, n):
    """Callers on either side of the path: count_if, inner_product, transform_reduce, the
    transform scans and scan_by_key (integer values, so every association order gives the
    same bits)."""
    x = datagen.c1_int32(n)
    y = datagen.c2_uint32(n).view(np.int32)
    out = {
        "c6.count_if_lt500": np.array([impl.count_if(x, LT, 500)], np.uint64),
        "c6.inner_product_i32_init11": np.array([impl.inner_product(x, y, init=11)], np.int32),
    }
    NEGATE, SQUARE, MAX = 1, 2, 2
    out["c6.transform_reduce_square_i32_init3"] = np.array([impl.transform_reduce(y, SQUARE, init=3)], np.int32)
    out["c6.transform_reduce_negate_max_i32"] = np.array([impl.transform_reduce(x, NEGATE, MAX, init=-2000)], np.int32)
    out["c6.transform_inclusive_scan_negate_i32"] = impl.transform_inclusive_scan(x, NEGATE)
    out["c6.transform_exclusive_scan_square_i32_init5"] = impl.transform_exclusive_scan(y, SQUARE, init=5)
    for mean in (8, 1000):
        k, v = datagen.c4_segments(n, mean)
        iv = (v * 1000).astype(np.int32)
        out[f"c6.m{mean}.inclusive_scan_by_key_i32"] = impl.inclusive_scan_by_key(k, iv)
        out[f"c6.m{mean}.exclusive_scan_by_key_i32_init9"] = impl.exclusive_scan_by_key(k, iv, init=9)
    return out


def c7(impl, n):
    """The four set operations on two sorted uint32 ranges with many repeated keys, and their
    by-key forms with the original index as value."""
    def sorted_with_index(count, seed, distinct):
        k = datagen.c2_uint32(count, seed) % np.uint32(distinct)
        order = np.argsort(k, kind="stable").astype(np.uint32)
        return k[order], order
    ka, va = sorted_with_index(n // 2, 8, n // 8 + 1)   # runs of about four equal keys
    kb, vb = sorted_with_index(n // 2, 9, n // 4 + 1)   # runs of about two, half the keys unmatched
    out = {}
    for op, name in enumerate(("difference", "intersection", "symmetric_difference", "union")):
        out[f"c7.set_{name}"] = impl.set_operation(op, ka, kb)
        k, v = impl.set_operation_by_key(op, ka, kb, va, vb)
        out[f"c7.set_{name}_by_key.values"] = v
    return out


def c8(impl, n):
    """The comparison sort (stable_sort with user-defined comparators: the reference's merge sort) and the
    reference's rules for mixed element types (conversions, accumulator of init's / the input's type)."""
    out = {}
    k = (datagen.c2_uint32(n) % np.uint32(1000)).astype(np.int32) - np.int32(500)
    f = datagen.c2_float32(n)  # with +0.0 / -0.0, equivalent under operator<: their input order must survive
    v = np.arange(n, dtype=np.uint32)
    out["c8.comparison_sort_i32"] = impl.comparison_sort(k)
    ko, vo = impl.comparison_sort(k, v, 1)
    out["c8.comparison_sort_by_key_i32_greater.values"] = vo
    ko, vo = impl.comparison_sort(f, v, 0)
    out["c8.comparison_sort_by_key_f32.key_bits"] = ko.view(np.uint32)
    out["c8.comparison_sort_by_key_f32.values"] = vo
    x = datagen.c1_int32(n)
    fx = x.astype(np.float32) / np.float32(4) - np.float32(100)
    out["c8.convert_f32_to_i32"] = impl.convert(fx, np.int32)
    out["c8.convert_i32_to_f32"] = impl.convert(x * np.int32(16777), np.float32)
    out["c8.reduce_f32_into_i32"] = np.array([impl.reduce_as(fx, np.int32(3))], np.int32)
    out["c8.inclusive_scan_i32_to_f32"] = impl.inclusive_scan_as(x, np.float32)
    out["c8.exclusive_scan_i32_init5_to_f32"] = impl.exclusive_scan_as(x, np.int32(5), np.float32)
    return out


CASES = {"c1": c1, "c2": c2, "c3": c3, "c4": c4, "c5": c5, "c6": c6, "c7": c7, "c8": c8}


def digest(a):
    a = np.ascontiguousarray(a)
    return hashlib.sha256(a.view(np.uint8).tobytes()).hexdigest()
