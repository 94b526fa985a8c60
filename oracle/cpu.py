"""TEST INFRASTRUCTURE -- numpy-facing binding of the CPU oracle and of the real reference.

`Oracle()`      loads oracle/libthrust_oracle.so, the C restatement (always available
                after `make -C oracle`).
`Reference(k)`  loads oracle/_ref/libref_{omp,cpp}.so, the real reference compiled from
                its own headers; available only where it was built (it needs the
                reference tree at build time, not at run time).
Both expose the same methods on numpy arrays and return new arrays; nothing here is
used by the library itself.
"""
import ctypes
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_LIB = os.path.join(HERE, "libthrust_oracle.so")
REF_LIBS = {"omp": os.path.join(HERE, "_ref", "libref_omp.so"),
            "cpp": os.path.join(HERE, "_ref", "libref_cpp.so")}

I8, U8, I16, U16, I32, U32, I64, U64, F32, F64 = range(10)
NP_DTYPES = {I8: np.int8, U8: np.uint8, I16: np.int16, U16: np.uint16, I32: np.int32,
             U32: np.uint32, I64: np.int64, U64: np.uint64, F32: np.float32, F64: np.float64}
DTYPE_OF_NP = {np.dtype(v): k for k, v in NP_DTYPES.items()}
PLUS, MIN, MAX = range(3)
LT, LE, GT, GE, EQ, NE, NONZERO = range(7)
CMP_SORT_LESS, CMP_SORT_GREATER, CMP_SORT_LESS_DIV = 0, 1, 2
IDENTITY, NEGATE, SQUARE = range(3)
SET_DIFFERENCE, SET_INTERSECTION, SET_SYMMETRIC_DIFFERENCE, SET_UNION = range(4)


def build(with_ref=True):
    """Runs oracle/Makefile (C restatement; the reference libraries where the tree exists)."""
    target = "all" if with_ref else os.path.join(HERE, "libthrust_oracle.so")
    subprocess.run(["make", "-C", HERE, "-j3", target], check=True, capture_output=True)


def ref_available(kind):
    return os.path.exists(REF_LIBS[kind])


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p) if a is not None else None


def _code(a):
    return DTYPE_OF_NP[a.dtype]


def _c(a):
    return np.ascontiguousarray(a)


class _Base:
    prefix = ""
    threaded = False

    def __init__(self, path):
        if not os.path.exists(path):
            raise FileNotFoundError(f"{path} is not built (make -C oracle)")
        self.lib = ctypes.CDLL(path)
        self.nthreads = 0  # 0 = library default (all cores); only the restatement honours it

    def _fn(self, name):
        fn = getattr(self.lib, self.prefix + name)
        fn.restype = ctypes.c_int
        return fn

    def _extra(self):
        return (ctypes.c_int(self.nthreads),) if self.threaded else ()

    @staticmethod
    def _ok(rc, what):
        if rc != 0:
            raise RuntimeError(f"{what} returned {rc}")

    def reduce(self, x, op=PLUS, init=0):
        x = _c(x)
        out = np.zeros(1, x.dtype)
        iv = np.array([init], x.dtype)
        self._ok(self._fn("reduce")(_p(x), ctypes.c_uint64(x.size), _code(x), op, _p(iv), _p(out),
                                     *self._extra()), "reduce")
        return out[0]

    def inclusive_scan(self, x, op=PLUS):
        x = _c(x)
        out = np.empty_like(x)
        self._ok(self._fn("inclusive_scan")(_p(x), _p(out), ctypes.c_uint64(x.size), _code(x), op),
                 "inclusive_scan")
        return out

    def exclusive_scan(self, x, init=0, op=PLUS):
        x = _c(x)
        out = np.empty_like(x)
        iv = np.array([init], x.dtype)
        self._ok(self._fn("exclusive_scan")(_p(x), _p(out), ctypes.c_uint64(x.size), _code(x), op,
                                             _p(iv)), "exclusive_scan")
        return out

    def sort_keys(self, keys, descending=False):
        k = _c(keys).copy()
        self._ok(self._fn("sort_keys")(_p(k), ctypes.c_uint64(k.size), _code(k), int(descending),
                                        *self._extra()), "sort_keys")
        return k

    def sort_pairs(self, keys, values, descending=False):
        k, v = _c(keys).copy(), _c(values).copy()
        self._ok(self._fn("sort_pairs")(_p(k), _p(v), ctypes.c_uint64(k.size), _code(k),
                                         ctypes.c_uint64(v.itemsize), int(descending),
                                         *self._extra()), "sort_pairs")
        return k, v

    def merge(self, a, b, descending=False):
        a, b = _c(a), _c(b)
        out = np.empty(a.size + b.size, a.dtype)
        self._ok(self._fn("merge")(_p(a), ctypes.c_uint64(a.size), _p(b), ctypes.c_uint64(b.size),
                                    _p(out), _code(a), int(descending)), "merge")
        return out

    def merge_by_key(self, ka, kb, va, vb, descending=False):
        ka, kb, va, vb = _c(ka), _c(kb), _c(va), _c(vb)
        ko = np.empty(ka.size + kb.size, ka.dtype)
        vo = np.empty(ka.size + kb.size, va.dtype)
        self._ok(self._fn("merge_by_key")(_p(ka), ctypes.c_uint64(ka.size), _p(kb),
                                           ctypes.c_uint64(kb.size), _p(va), _p(vb), _p(ko), _p(vo),
                                           _code(ka), ctypes.c_uint64(va.itemsize),
                                           int(descending)), "merge_by_key")
        return ko, vo

    def copy_if(self, x, cmp, threshold=0, stencil=None):
        x = _c(x)
        st = _c(stencil) if stencil is not None else None
        tested = st if st is not None else x
        out = np.empty_like(x)
        num = ctypes.c_uint64(0)
        tv = np.array([threshold], tested.dtype)
        self._ok(self._fn("copy_if")(_p(x), _p(st), _p(out), ctypes.byref(num),
                                      ctypes.c_uint64(x.size), ctypes.c_uint64(x.itemsize),
                                      _code(tested), cmp, _p(tv)), "copy_if")
        return out[: num.value].copy()

    def partition_copy(self, x, cmp, threshold=0, stencil=None):
        x = _c(x)
        st = _c(stencil) if stencil is not None else None
        tested = st if st is not None else x
        ot, of = np.empty_like(x), np.empty_like(x)
        num = ctypes.c_uint64(0)
        tv = np.array([threshold], tested.dtype)
        self._ok(self._fn("partition_copy")(_p(x), _p(st), _p(ot), _p(of), ctypes.byref(num),
                                             ctypes.c_uint64(x.size), ctypes.c_uint64(x.itemsize),
                                             _code(tested), cmp, _p(tv)), "partition_copy")
        t = num.value
        return ot[:t].copy(), of[: x.size - t].copy()

    def stable_partition(self, x, cmp, threshold=0, stencil=None):
        x = _c(x).copy()
        st = _c(stencil) if stencil is not None else None
        tested = st if st is not None else x
        num = ctypes.c_uint64(0)
        tv = np.array([threshold], tested.dtype)
        self._ok(self._fn("stable_partition")(_p(x), _p(st), ctypes.byref(num),
                                               ctypes.c_uint64(x.size), ctypes.c_uint64(x.itemsize),
                                               _code(tested), cmp, _p(tv)), "stable_partition")
        return x, num.value

    def unique(self, x):
        x = _c(x)
        out = np.empty_like(x)
        num = ctypes.c_uint64(0)
        self._ok(self._fn("unique")(_p(x), _p(out), ctypes.byref(num), ctypes.c_uint64(x.size),
                                     _code(x)), "unique")
        return out[: num.value].copy()

    def unique_by_key(self, keys, values):
        k, v = _c(keys), _c(values)
        ko, vo = np.empty_like(k), np.empty_like(v)
        num = ctypes.c_uint64(0)
        self._ok(self._fn("unique_by_key")(_p(k), _p(v), _p(ko), _p(vo), ctypes.byref(num),
                                            ctypes.c_uint64(k.size), _code(k),
                                            ctypes.c_uint64(v.itemsize)), "unique_by_key")
        return ko[: num.value].copy(), vo[: num.value].copy()

    def reduce_by_key(self, keys, values, op=PLUS):
        k, v = _c(keys), _c(values)
        ko, vo = np.empty_like(k), np.empty_like(v)
        num = ctypes.c_uint64(0)
        self._ok(self._fn("reduce_by_key")(_p(k), _p(v), _p(ko), _p(vo), ctypes.byref(num),
                                            ctypes.c_uint64(k.size), _code(k), _code(v), op),
                 "reduce_by_key")
        return ko[: num.value].copy(), vo[: num.value].copy()

    def count_if(self, x, cmp, threshold=0):
        x = _c(x)
        num = ctypes.c_uint64(0)
        tv = np.array([threshold], x.dtype)
        self._ok(self._fn("count_if")(_p(x), ctypes.c_uint64(x.size), _code(x), cmp, _p(tv),
                                       ctypes.byref(num), *self._extra()), "count_if")
        return num.value

    def inner_product(self, a, b, init=0):
        a, b = _c(a), _c(b)
        out = np.zeros(1, a.dtype)
        iv = np.array([init], a.dtype)
        self._ok(self._fn("inner_product")(_p(a), _p(b), ctypes.c_uint64(a.size), _code(a), _p(iv),
                                            _p(out), *self._extra()), "inner_product")
        return out[0]

    def convert(self, x, dtype):
        x = _c(x)
        out = np.empty(x.size, dtype)
        self._ok(self._fn("convert")(_p(x), _code(x), _p(out), _code(out), ctypes.c_uint64(x.size)), "convert")
        return out

    # The reference's type rules for mixed element types (see oracle_convert).
    def reduce_as(self, x, init, op=PLUS):
        """reduce(first, last, init): the accumulator has init's type."""
        init = np.asarray(init)
        return self.reduce(self.convert(x, init.dtype), op, init[()])

    def inclusive_scan_as(self, x, out_dtype, op=PLUS):
        """inclusive_scan(first, last, result): accumulates in the input's type, converts on output."""
        return self.convert(self.inclusive_scan(x, op), out_dtype)

    def exclusive_scan_as(self, x, init, out_dtype, op=PLUS):
        """exclusive_scan(first, last, result, init): accumulates in init's type, converts on output."""
        init = np.asarray(init)
        return self.convert(self.exclusive_scan(self.convert(x, init.dtype), init[()], op), out_dtype)

    def comparison_sort(self, keys, values=None, comparator=CMP_SORT_LESS, param=0):
        """stable_sort(_by_key) with a user comparator: returns sorted copies."""
        k = _c(keys).copy()
        v = None if values is None else _c(values).copy()
        self._ok(self._fn("comparison_sort")(_p(k), _p(v) if v is not None else None, ctypes.c_uint64(k.size),
                                              _code(k), ctypes.c_uint64(0 if v is None else v.itemsize),
                                              int(comparator), ctypes.c_long(int(param))), "comparison_sort")
        return k if v is None else (k, v)

    def set_operation(self, op, a, b, descending=False):
        a, b = _c(a), _c(b)
        out = np.empty(a.size + b.size, a.dtype)
        num = ctypes.c_uint64(0)
        self._ok(self._fn("set_operation")(op, _p(a), ctypes.c_uint64(a.size), _p(b), ctypes.c_uint64(b.size),
                                            _p(out), ctypes.byref(num), _code(a), int(descending)),
                 "set_operation")
        return out[: num.value].copy()

    def set_operation_by_key(self, op, ka, kb, va, vb, descending=False):
        ka, kb, va, vb = _c(ka), _c(kb), _c(va), _c(vb)
        ko = np.empty(ka.size + kb.size, ka.dtype)
        vo = np.empty(ka.size + kb.size, va.dtype)
        num = ctypes.c_uint64(0)
        self._ok(self._fn("set_operation_by_key")(op, _p(ka), ctypes.c_uint64(ka.size), _p(kb),
                                                   ctypes.c_uint64(kb.size), _p(va), _p(vb), _p(ko), _p(vo),
                                                   ctypes.byref(num), _code(ka), ctypes.c_uint64(va.itemsize),
                                                   int(descending)), "set_operation_by_key")
        return ko[: num.value].copy(), vo[: num.value].copy()

    def transform_reduce(self, x, unary, op=PLUS, init=0):
        x = _c(x)
        out = np.zeros(1, x.dtype)
        iv = np.array([init], x.dtype)
        self._ok(self._fn("transform_reduce")(_p(x), ctypes.c_uint64(x.size), _code(x), unary, op,
                                               _p(iv), _p(out), *self._extra()), "transform_reduce")
        return out[0]

    def transform_inclusive_scan(self, x, unary, op=PLUS):
        x = _c(x)
        out = np.empty_like(x)
        self._ok(self._fn("transform_inclusive_scan")(_p(x), _p(out), ctypes.c_uint64(x.size),
                                                       _code(x), unary, op), "transform_inclusive_scan")
        return out

    def transform_exclusive_scan(self, x, unary, init=0, op=PLUS):
        x = _c(x)
        out = np.empty_like(x)
        iv = np.array([init], x.dtype)
        self._ok(self._fn("transform_exclusive_scan")(_p(x), _p(out), ctypes.c_uint64(x.size),
                                                       _code(x), unary, op, _p(iv)),
                 "transform_exclusive_scan")
        return out

    def inclusive_scan_by_key(self, keys, values, op=PLUS):
        k, v = _c(keys), _c(values)
        out = np.empty_like(v)
        self._ok(self._fn("inclusive_scan_by_key")(_p(k), _p(v), _p(out), ctypes.c_uint64(k.size),
                                                    _code(k), _code(v), op), "inclusive_scan_by_key")
        return out

    def exclusive_scan_by_key(self, keys, values, init=0, op=PLUS):
        k, v = _c(keys), _c(values)
        out = np.empty_like(v)
        iv = np.array([init], v.dtype)
        self._ok(self._fn("exclusive_scan_by_key")(_p(k), _p(v), _p(out), ctypes.c_uint64(k.size),
                                                    _code(k), _code(v), op, _p(iv)),
                 "exclusive_scan_by_key")
        return out


class Oracle(_Base):
    """The C restatement.  `nthreads` (0 = all cores) sets the OMP shape; 1 = CPP system."""
    prefix = "oracle_"
    threaded = True

    def __init__(self, nthreads=0):
        super().__init__(ORACLE_LIB)
        self.nthreads = nthreads

    def decompose(self, n, granularity, max_intervals):
        b = (ctypes.c_long * max(max_intervals, 1))()
        e = (ctypes.c_long * max(max_intervals, 1))()
        fn = self.lib.oracle_decompose
        fn.restype = ctypes.c_long
        k = fn(ctypes.c_long(n), ctypes.c_long(granularity), ctypes.c_long(max_intervals), b, e)
        return [(b[i], e[i]) for i in range(k)]


class Reference(_Base):
    """The real reference, kind = "omp" or "cpp"."""
    prefix = "ref_"
    threaded = False

    def __init__(self, kind, path=None):
        """path: another build of ref_driver.cpp with the same exports (the tests compile it
        against this repository's own headers to check their host system)."""
        super().__init__(path or REF_LIBS[kind])
        self.kind = kind

    # The real mixed-type calls, int32 <-> float32 only: these run the reference's own type
    # deduction, where the methods of the same names above restate it with conversions.
    def reduce_as(self, x, init, op=PLUS):
        x, init = _c(x), np.asarray(init)
        if op != PLUS:
            raise ValueError("the reference driver instantiates plus only for mixed types")
        iv, out = np.array([init], init.dtype), np.empty(1, init.dtype)
        self._ok(self._fn("reduce_mixed")(_p(x), _code(x), ctypes.c_uint64(x.size), _code(iv), _p(iv), _p(out)),
                 "reduce_mixed")
        return out[0]

    # thrust::shuffle_copy / thrust::shuffle with thrust::default_random_engine(seed).
    def shuffle_copy(self, x, seed):
        x = _c(x)
        out = np.empty_like(x)
        self._ok(self._fn("shuffle_copy")(_p(x), _p(out), ctypes.c_uint64(x.size), _code(x), ctypes.c_uint32(seed)),
                 "shuffle_copy")
        return out

    def shuffle(self, x, seed):
        out = _c(x).copy()
        self._ok(self._fn("shuffle")(_p(out), ctypes.c_uint64(out.size), _code(out), ctypes.c_uint32(seed)), "shuffle")
        return out

    def _scan_mixed(self, x, out_dtype, exclusive, init):
        x = _c(x)
        out = np.empty(x.size, out_dtype)
        if {x.dtype, out.dtype} != {np.dtype(np.int32), np.dtype(np.float32)}:
            raise ValueError("the reference driver instantiates int32 <-> float32 only")
        iv = np.array([0 if init is None else init], np.int32 if init is None else np.asarray(init).dtype)
        self._ok(self._fn("scan_mixed")(_p(x), _code(x), _p(out), ctypes.c_uint64(x.size), exclusive, _code(iv),
                                        _p(iv)), "scan_mixed")
        return out

    def inclusive_scan_as(self, x, out_dtype, op=PLUS):
        return self._scan_mixed(x, out_dtype, -1, None)

    def exclusive_scan_as(self, x, init, out_dtype, op=PLUS):
        return self._scan_mixed(x, out_dtype, 1, init)
