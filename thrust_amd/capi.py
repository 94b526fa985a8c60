"""ctypes binding of libthrust_amd.so (the C ABI declared in include/thrust_amd.h).

This module is plumbing for tests and the benchmark: it loads the in-tree shared
library, declares the argument types of every entry point and offers thin helpers that
run the two-phase temp-storage protocol on torch-owned device memory.  There is no
fallback: if the library is missing or an entry point fails, an exception is raised.
"""
import ctypes
import os

import numpy as np

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(PKG_DIR, "libthrust_amd.so")

# dtype codes (thrust_amd_dtype)
I8, U8, I16, U16, I32, U32, I64, U64, F32, F64 = range(10)
NP_DTYPES = {
    I8: np.int8, U8: np.uint8, I16: np.int16, U16: np.uint16, I32: np.int32,
    U32: np.uint32, I64: np.int64, U64: np.uint64, F32: np.float32, F64: np.float64,
}
DTYPE_OF_NP = {np.dtype(v): k for k, v in NP_DTYPES.items()}
DTYPE_NAMES = {I8: "i8", U8: "u8", I16: "i16", U16: "u16", I32: "i32", U32: "u32",
               I64: "i64", U64: "u64", F32: "f32", F64: "f64"}
# thrust_amd_binop
PLUS, MIN, MAX = range(3)
# thrust_amd_cmp
LT, LE, GT, GE, EQ, NE, NONZERO = range(7)
IDENTITY, NEGATE, SQUARE = range(3)
SET_DIFFERENCE, SET_INTERSECTION, SET_SYMMETRIC_DIFFERENCE, SET_UNION = range(4)
H2D, D2H, D2D = 1, 2, 3

_c = ctypes
_vp, _sz, _u64, _int = _c.c_void_p, _c.c_size_t, _c.c_uint64, _c.c_int
_szp = _c.POINTER(_c.c_size_t)

# name -> (restype, argtypes); must list every function include/thrust_amd.h declares.
SIGNATURES = {
    "thrust_amd_version": (_int, []),
    "thrust_amd_error_string": (_c.c_char_p, [_int]),
    "thrust_amd_dtype_size": (_sz, [_int]),
    "thrust_amd_malloc": (_int, [_c.POINTER(_vp), _sz]),
    "thrust_amd_free": (_int, [_vp]),
    "thrust_amd_memcpy": (_int, [_vp, _vp, _sz, _int, _vp]),
    "thrust_amd_stream_synchronize": (_int, [_vp]),
    "thrust_amd_fill": (_int, [_vp, _u64, _sz, _vp, _vp]),
    "thrust_amd_temp_acquire": (_int, [_c.POINTER(_vp), _sz, _vp]),
    "thrust_amd_temp_release": (_int, [_vp, _vp]),
    "thrust_amd_temp_trim": (_int, []),
    "thrust_amd_temp_bytes_held": (_sz, []),
    "thrust_amd_profile_enable": (_int, [_int]),
    "thrust_amd_profile_collect": (_int, [_c.c_char_p, _sz, _szp]),
    "thrust_amd_convert": (_int, [_vp, _int, _vp, _int, _u64, _vp]),
    "thrust_amd_sequence": (_int, [_vp, _u64, _int, _vp, _vp, _vp]),
    "thrust_amd_stream_create": (_int, [ctypes.POINTER(_vp)]),
    "thrust_amd_stream_destroy": (_int, [_vp]),
    "thrust_amd_stream_query": (_int, [_vp, ctypes.POINTER(_int)]),
    "thrust_amd_event_create": (_int, [ctypes.POINTER(_vp)]),
    "thrust_amd_event_record": (_int, [_vp, _vp]),
    "thrust_amd_stream_wait_event": (_int, [_vp, _vp]),
    "thrust_amd_event_destroy": (_int, [_vp]),
    "thrust_amd_reduce": (_int, [_vp, _szp, _vp, _u64, _int, _int, _vp, _vp, _vp]),
    "thrust_amd_transform_reduce": (_int, [_vp, _szp, _vp, _u64, _int, _int, _int, _vp, _vp, _vp]),
    "thrust_amd_count_if": (_int, [_vp, _szp, _vp, _u64, _int, _int, _vp, _vp, _vp]),
    "thrust_amd_inner_product": (_int, [_vp, _szp, _vp, _vp, _u64, _int, _vp, _vp, _vp]),
    "thrust_amd_inclusive_scan": (_int, [_vp, _szp, _vp, _vp, _u64, _int, _int, _vp]),
    "thrust_amd_inclusive_scan_static": (_int, [_vp, _vp, _u64, _int, _int, _vp]),
    "thrust_amd_exclusive_scan": (_int, [_vp, _szp, _vp, _vp, _u64, _int, _int, _vp, _vp]),
    "thrust_amd_transform_inclusive_scan": (_int, [_vp, _szp, _vp, _vp, _u64, _int, _int, _int, _vp]),
    "thrust_amd_transform_exclusive_scan": (_int, [_vp, _szp, _vp, _vp, _u64, _int, _int, _int, _vp, _vp]),
    "thrust_amd_inclusive_scan_by_key": (_int, [_vp, _szp, _vp, _vp, _vp, _u64, _int, _int, _int, _vp]),
    "thrust_amd_exclusive_scan_by_key": (_int, [_vp, _szp, _vp, _vp, _vp, _u64, _int, _int, _int, _vp, _vp]),
    "thrust_amd_set_operation": (_int, [_vp, _szp, _int, _vp, _u64, _vp, _u64, _vp, _vp, _int, _int, _vp]),
    "thrust_amd_set_operation_by_key": (_int, [_vp, _szp, _int, _vp, _u64, _vp, _u64, _vp, _vp, _vp, _vp, _vp,
                                               _int, _sz, _int, _vp]),
    "thrust_amd_sort_keys": (_int, [_vp, _szp, _vp, _u64, _int, _int, _int, _int, _vp]),
    "thrust_amd_sort_pairs": (_int, [_vp, _szp, _vp, _vp, _u64, _int, _sz, _int, _int, _int, _vp]),
    "thrust_amd_malloc_universal": (_int, [_c.POINTER(_vp), _sz]),
    "thrust_amd_free_universal": (_int, [_vp]),
    "thrust_amd_merge_sort_keys": (_int, [_vp, _szp, _vp, _u64, _int, _int, _vp]),
    "thrust_amd_merge_sort_pairs": (_int, [_vp, _szp, _vp, _vp, _u64, _int, _sz, _int, _vp]),
    "thrust_amd_copy_if": (_int, [_vp, _szp, _vp, _vp, _vp, _vp, _u64, _sz, _int, _int, _vp, _vp]),
    "thrust_amd_partition_copy": (_int, [_vp, _szp, _vp, _vp, _vp, _vp, _vp, _u64, _sz, _int, _int, _vp, _vp]),
    "thrust_amd_stable_partition": (_int, [_vp, _szp, _vp, _vp, _vp, _u64, _sz, _int, _int, _vp, _vp]),
    "thrust_amd_unique": (_int, [_vp, _szp, _vp, _vp, _vp, _u64, _int, _vp]),
    "thrust_amd_unique_by_key": (_int, [_vp, _szp, _vp, _vp, _vp, _vp, _vp, _u64, _int, _sz, _vp]),
    "thrust_amd_reduce_by_key": (_int, [_vp, _szp, _vp, _vp, _vp, _vp, _vp, _u64, _int, _int, _int, _vp]),
    "thrust_amd_merge": (_int, [_vp, _szp, _vp, _u64, _vp, _u64, _vp, _int, _int, _vp]),
    "thrust_amd_merge_by_key": (_int, [_vp, _szp, _vp, _u64, _vp, _u64, _vp, _vp, _vp, _vp, _int, _sz, _int, _vp]),
}

_lib = None


class ThrustAmdError(RuntimeError):
    pass


def load():
    """Loads libthrust_amd.so (once) and declares all signatures.  Raises if it is missing."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ThrustAmdError(
            f"{LIB_PATH} is missing: build it with `python -m thrust_amd.build` "
            "(there is no fallback path)")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(status, what):
    if status != 0:
        msg = load().thrust_amd_error_string(status).decode()
        raise ThrustAmdError(f"{what} failed with status {status}: {msg}")


# ----------------------------------------------------------------- device-side helpers
def _torch():
    import torch
    return torch


class DeviceArray:
    """n elements of a C-ABI dtype in device memory owned by a torch uint8 tensor."""

    def __init__(self, n, dtype, storage=None):
        torch = _torch()
        self.n = int(n)
        self.dtype = dtype
        self.itemsize = np.dtype(NP_DTYPES[dtype]).itemsize
        nbytes = max(self.n * self.itemsize, 16)
        self.storage = storage if storage is not None else torch.empty(
            nbytes, dtype=torch.uint8, device="cuda")

    @property
    def ptr(self):
        return self.storage.data_ptr()

    @classmethod
    def from_numpy(cls, a):
        torch = _torch()
        a = np.ascontiguousarray(a)
        d = cls(a.size, DTYPE_OF_NP[a.dtype])
        if a.size:
            d.storage[: a.nbytes].copy_(torch.from_numpy(a.reshape(-1).view(np.uint8)))
        return d

    def numpy(self, count=None):
        count = self.n if count is None else int(count)
        nbytes = count * self.itemsize
        host = self.storage[:nbytes].cpu().numpy()
        return host.view(NP_DTYPES[self.dtype]).copy()

    def clone(self):
        return DeviceArray(self.n, self.dtype, self.storage.clone())


def stream_ptr():
    return _torch().cuda.current_stream().cuda_stream


def _scalar(dtype, value):
    return np.array([value], dtype=NP_DTYPES[dtype])


class Temp:
    """Temp storage for one entry point: size query, then a torch-owned buffer."""

    def __init__(self):
        self.buf = None
        self.bytes = ctypes.c_size_t(0)

    def ensure(self, query):
        """query(temp_ptr, byref(bytes)) -> status; runs the size query and allocates."""
        torch = _torch()
        self.bytes = ctypes.c_size_t(0)
        check(query(None, ctypes.byref(self.bytes)), "temp size query")
        need = max(int(self.bytes.value), 256)
        if self.buf is None or self.buf.numel() < need:
            self.buf = torch.empty(need, dtype=torch.uint8, device="cuda")
        return self.buf.data_ptr()


def _run(fn_name, temp, call):
    lib = load()
    fn = getattr(lib, fn_name)
    temp = temp or Temp()
    tptr = temp.ensure(lambda t, b: call(fn, t, b))
    check(call(fn, tptr, ctypes.byref(temp.bytes)), fn_name)
    return temp


def profile_enable(on=True):
    check(load().thrust_amd_profile_enable(int(on)), "profile_enable")


def profile_collect():
    """Returns {label: (launches, total_ms)} for the kernels launched since the last call."""
    lib = load()
    buf = ctypes.create_string_buffer(1 << 16)
    need = ctypes.c_size_t(0)
    check(lib.thrust_amd_profile_collect(buf, len(buf), ctypes.byref(need)), "profile_collect")
    out = {}
    for line in buf.value.decode().splitlines():
        label, launches, ms = line.split()
        out[label] = (int(launches), float(ms))
    return out


def reduce(x, op=PLUS, init=0, temp=None, out=None):
    out = out or DeviceArray(1, x.dtype)
    iv = _scalar(x.dtype, init)
    _run("thrust_amd_reduce", temp, lambda fn, t, b: fn(
        t, b, x.ptr, x.n, x.dtype, op, iv.ctypes.data, out.ptr, stream_ptr()))
    return out


def convert(x, out_dtype, out=None):
    out = out or DeviceArray(x.n, out_dtype)
    check(load().thrust_amd_convert(x.ptr, x.dtype, out.ptr, out_dtype, x.n, stream_ptr()), "thrust_amd_convert")
    return out


def sequence(n, dtype, init=0, step=1, out=None):
    out = out or DeviceArray(n, dtype)
    iv, sv = _scalar(dtype, init), _scalar(dtype, step)
    check(load().thrust_amd_sequence(out.ptr, n, dtype, iv.ctypes.data, sv.ctypes.data, stream_ptr()), "thrust_amd_sequence")
    return out


def transform_reduce(x, unary, op=PLUS, init=0, temp=None, out=None):
    out = out or DeviceArray(1, x.dtype)
    iv = _scalar(x.dtype, init)
    _run("thrust_amd_transform_reduce", temp, lambda fn, t, b: fn(
        t, b, x.ptr, x.n, x.dtype, unary, op, iv.ctypes.data, out.ptr, stream_ptr()))
    return out


def count_if(x, cmp, threshold=0, temp=None, read_count=True):
    num = DeviceArray(1, U64)
    tv = _scalar(x.dtype, threshold)
    _run("thrust_amd_count_if", temp, lambda fn, t, b: fn(
        t, b, x.ptr, x.n, x.dtype, cmp, tv.ctypes.data, num.ptr, stream_ptr()))
    return _count(num, read_count)


def inner_product(a, b_, init=0, temp=None, out=None):
    out = out or DeviceArray(1, a.dtype)
    iv = _scalar(a.dtype, init)
    _run("thrust_amd_inner_product", temp, lambda fn, t, b: fn(
        t, b, a.ptr, b_.ptr, a.n, a.dtype, iv.ctypes.data, out.ptr, stream_ptr()))
    return out


def inclusive_scan(x, out=None, op=PLUS, temp=None):
    out = out or DeviceArray(x.n, x.dtype)
    _run("thrust_amd_inclusive_scan", temp, lambda fn, t, b: fn(
        t, b, x.ptr, out.ptr, x.n, x.dtype, op, stream_ptr()))
    return out


def inclusive_scan_static(x, out=None, op=PLUS):
    """The allocation-free entry point: no temp argument at all."""
    out = out or DeviceArray(x.n, x.dtype)
    check(load().thrust_amd_inclusive_scan_static(x.ptr, out.ptr, x.n, x.dtype, op, stream_ptr()),
          "thrust_amd_inclusive_scan_static")
    return out


def exclusive_scan(x, init=0, out=None, op=PLUS, temp=None):
    out = out or DeviceArray(x.n, x.dtype)
    iv = _scalar(x.dtype, init)
    _run("thrust_amd_exclusive_scan", temp, lambda fn, t, b: fn(
        t, b, x.ptr, out.ptr, x.n, x.dtype, op, iv.ctypes.data, stream_ptr()))
    return out


def transform_inclusive_scan(x, unary, out=None, op=PLUS, temp=None):
    out = out or DeviceArray(x.n, x.dtype)
    _run("thrust_amd_transform_inclusive_scan", temp, lambda fn, t, b: fn(
        t, b, x.ptr, out.ptr, x.n, x.dtype, unary, op, stream_ptr()))
    return out


def transform_exclusive_scan(x, unary, init=0, out=None, op=PLUS, temp=None):
    out = out or DeviceArray(x.n, x.dtype)
    iv = _scalar(x.dtype, init)
    _run("thrust_amd_transform_exclusive_scan", temp, lambda fn, t, b: fn(
        t, b, x.ptr, out.ptr, x.n, x.dtype, unary, op, iv.ctypes.data, stream_ptr()))
    return out


def inclusive_scan_by_key(keys, values, op=PLUS, out=None, temp=None):
    out = out or DeviceArray(values.n, values.dtype)
    _run("thrust_amd_inclusive_scan_by_key", temp, lambda fn, t, b: fn(
        t, b, keys.ptr, values.ptr, out.ptr, keys.n, keys.dtype, values.dtype, op, stream_ptr()))
    return out


def exclusive_scan_by_key(keys, values, init=0, op=PLUS, out=None, temp=None):
    out = out or DeviceArray(values.n, values.dtype)
    iv = _scalar(values.dtype, init)
    _run("thrust_amd_exclusive_scan_by_key", temp, lambda fn, t, b: fn(
        t, b, keys.ptr, values.ptr, out.ptr, keys.n, keys.dtype, values.dtype, op, iv.ctypes.data,
        stream_ptr()))
    return out


def sort_keys(keys, descending=False, begin_bit=0, end_bit=None, temp=None):
    end_bit = keys.itemsize * 8 if end_bit is None else end_bit
    return _run("thrust_amd_sort_keys", temp, lambda fn, t, b: fn(
        t, b, keys.ptr, keys.n, keys.dtype, int(descending), begin_bit, end_bit, stream_ptr()))


def sort_pairs(keys, values, descending=False, begin_bit=0, end_bit=None, temp=None):
    end_bit = keys.itemsize * 8 if end_bit is None else end_bit
    return _run("thrust_amd_sort_pairs", temp, lambda fn, t, b: fn(
        t, b, keys.ptr, values.ptr, keys.n, keys.dtype, values.itemsize, int(descending),
        begin_bit, end_bit, stream_ptr()))


def merge_sort_keys(keys, descending=False, temp=None):
    """Stable comparison sort in place (operator< / operator>)."""
    return _run("thrust_amd_merge_sort_keys", temp, lambda fn, t, b: fn(
        t, b, keys.ptr, keys.n, keys.dtype, int(descending), stream_ptr()))


def merge_sort_pairs(keys, values, descending=False, temp=None):
    return _run("thrust_amd_merge_sort_pairs", temp, lambda fn, t, b: fn(
        t, b, keys.ptr, values.ptr, keys.n, keys.dtype, values.itemsize, int(descending), stream_ptr()))


def _count(dev_u64, read=True):
    """The uint64 result count: read back (blocks) or, with read=False, left on the device
    for callers that must not synchronise inside a timed region."""
    return int(dev_u64.numpy()[0]) if read else dev_u64


def copy_if(x, cmp, threshold=0, stencil=None, out=None, temp=None, read_count=True):
    out = out or DeviceArray(x.n, x.dtype)
    num = DeviceArray(1, U64)
    tested = stencil if stencil is not None else x
    tv = _scalar(tested.dtype, threshold)
    _run("thrust_amd_copy_if", temp, lambda fn, t, b: fn(
        t, b, x.ptr, stencil.ptr if stencil is not None else None, out.ptr, num.ptr, x.n,
        x.itemsize, tested.dtype, cmp, tv.ctypes.data, stream_ptr()))
    return out, _count(num, read_count)


def partition_copy(x, cmp, threshold=0, stencil=None, temp=None, read_count=True):
    out_t, out_f = DeviceArray(x.n, x.dtype), DeviceArray(x.n, x.dtype)
    num = DeviceArray(1, U64)
    tested = stencil if stencil is not None else x
    tv = _scalar(tested.dtype, threshold)
    _run("thrust_amd_partition_copy", temp, lambda fn, t, b: fn(
        t, b, x.ptr, stencil.ptr if stencil is not None else None, out_t.ptr, out_f.ptr, num.ptr,
        x.n, x.itemsize, tested.dtype, cmp, tv.ctypes.data, stream_ptr()))
    return out_t, out_f, _count(num, read_count)


def stable_partition(x, cmp, threshold=0, stencil=None, temp=None, read_count=True):
    num = DeviceArray(1, U64)
    tested = stencil if stencil is not None else x
    tv = _scalar(tested.dtype, threshold)
    _run("thrust_amd_stable_partition", temp, lambda fn, t, b: fn(
        t, b, x.ptr, stencil.ptr if stencil is not None else None, num.ptr, x.n, x.itemsize,
        tested.dtype, cmp, tv.ctypes.data, stream_ptr()))
    return _count(num, read_count)


def unique(x, out=None, temp=None, read_count=True):
    out = out or DeviceArray(x.n, x.dtype)
    num = DeviceArray(1, U64)
    _run("thrust_amd_unique", temp, lambda fn, t, b: fn(
        t, b, x.ptr, out.ptr, num.ptr, x.n, x.dtype, stream_ptr()))
    return out, _count(num, read_count)


def unique_by_key(keys, values, keys_out=None, values_out=None, temp=None, read_count=True):
    keys_out = keys_out or DeviceArray(keys.n, keys.dtype)
    values_out = values_out or DeviceArray(values.n, values.dtype)
    num = DeviceArray(1, U64)
    _run("thrust_amd_unique_by_key", temp, lambda fn, t, b: fn(
        t, b, keys.ptr, values.ptr, keys_out.ptr, values_out.ptr, num.ptr, keys.n, keys.dtype,
        values.itemsize, stream_ptr()))
    return keys_out, values_out, _count(num, read_count)


def reduce_by_key(keys, values, op=PLUS, temp=None, keys_out=None, values_out=None, read_count=True):
    keys_out = keys_out or DeviceArray(keys.n, keys.dtype)
    values_out = values_out or DeviceArray(values.n, values.dtype)
    num = DeviceArray(1, U64)
    _run("thrust_amd_reduce_by_key", temp, lambda fn, t, b: fn(
        t, b, keys.ptr, values.ptr, keys_out.ptr, values_out.ptr, num.ptr, keys.n, keys.dtype,
        values.dtype, op, stream_ptr()))
    return keys_out, values_out, _count(num, read_count)


def merge(a, b_, descending=False, out=None, temp=None):
    out = out or DeviceArray(a.n + b_.n, a.dtype)
    _run("thrust_amd_merge", temp, lambda fn, t, b: fn(
        t, b, a.ptr, a.n, b_.ptr, b_.n, out.ptr, a.dtype, int(descending), stream_ptr()))
    return out


def set_operation(op, a, b_, descending=False, out=None, temp=None, read_count=True):
    """Returns (out, length); out holds a.n + b.n elements unless the caller passes one."""
    out = out or DeviceArray(a.n + b_.n, a.dtype)
    num = DeviceArray(1, U64)
    _run("thrust_amd_set_operation", temp, lambda fn, t, b: fn(
        t, b, op, a.ptr, a.n, b_.ptr, b_.n, out.ptr, num.ptr, a.dtype, int(descending), stream_ptr()))
    return out, _count(num, read_count)


def set_operation_by_key(op, ka, kb, va, vb, descending=False, temp=None, keys_out=None, values_out=None, read_count=True):
    keys_out = keys_out or DeviceArray(ka.n + kb.n, ka.dtype)
    values_out = values_out or DeviceArray(ka.n + kb.n, va.dtype)
    num = DeviceArray(1, U64)
    _run("thrust_amd_set_operation_by_key", temp, lambda fn, t, b: fn(
        t, b, op, ka.ptr, ka.n, kb.ptr, kb.n, va.ptr, vb.ptr if vb is not None else None, keys_out.ptr,
        values_out.ptr, num.ptr, ka.dtype, va.itemsize, int(descending), stream_ptr()))
    return keys_out, values_out, _count(num, read_count)


def merge_by_key(ka, kb, va, vb, descending=False, temp=None, keys_out=None, values_out=None):
    keys_out = keys_out or DeviceArray(ka.n + kb.n, ka.dtype)
    values_out = values_out or DeviceArray(ka.n + kb.n, va.dtype)
    _run("thrust_amd_merge_by_key", temp, lambda fn, t, b: fn(
        t, b, ka.ptr, ka.n, kb.ptr, kb.n, va.ptr, vb.ptr, keys_out.ptr, values_out.ptr, ka.dtype,
        va.itemsize, int(descending), stream_ptr()))
    return keys_out, values_out
