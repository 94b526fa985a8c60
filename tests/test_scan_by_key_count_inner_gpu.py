"""GPU parity: thrust_amd_inclusive/exclusive_scan_by_key, thrust_amd_count_if and
thrust_amd_inner_product against the CPU oracle.

Integer results are exact for every association order (wrap-around arithmetic is
associative and commutative); float32 results are compared with the oracle's strict
left fold within 1e-5 relative and with a float64 fold.  Models:
testing/scan_by_key.cu:23-220 (segments, init, in place), testing/count.cu:33-60,
testing/inner_product.cu:9-62.
"""
import numpy as np
import pytest

from thrust_amd import datagen

pytestmark = pytest.mark.gpu

SIZES = [0, 1, 2, 63, 64, 65, 1000, 16383, 16384, 16385, 32769, 100003, (1 << 20) + 13]
REL_TOL = 1e-5
INT_DTYPES = [np.int8, np.uint8, np.int16, np.uint16, np.int32, np.uint32, np.int64, np.uint64]


def _keys(n, dtype, seed, mean):
    lens = (datagen.splitmix64(seed, n) % np.uint64(2 * mean)).astype(np.int64) + 1
    ids = np.repeat(np.arange(n, dtype=np.int64), lens)[:n]
    vals = (datagen.splitmix64(seed + 1, n) % np.uint64(97)).astype(np.int64)
    return vals[ids].astype(dtype)


@pytest.mark.parametrize("kdtype", [np.int32, np.uint8, np.int64, np.uint16, np.float32, np.float64])
@pytest.mark.parametrize("vdtype", [np.int32, np.uint64, np.int8, np.int16])
def test_scan_by_key_integer_values_exact(dev, oracle, kdtype, vdtype):
    for n in SIZES:
        k = _keys(n, kdtype, 3, 5)
        v = (datagen.splitmix64(9, n) >> np.uint64(20)).astype(vdtype)
        dk, dv = dev.DeviceArray.from_numpy(k), dev.DeviceArray.from_numpy(v)
        got = dev.inclusive_scan_by_key(dk, dv).numpy()
        assert np.array_equal(got, oracle.inclusive_scan_by_key(k, v)), ("inclusive", kdtype, vdtype, n)
        got = dev.exclusive_scan_by_key(dk, dv, init=7).numpy()
        assert np.array_equal(got, oracle.exclusive_scan_by_key(k, v, init=7)), ("exclusive", kdtype, vdtype, n)


@pytest.mark.parametrize("op", [1, 2])
def test_scan_by_key_min_max(dev, oracle, op):
    n = 70001
    k = _keys(n, np.int32, 5, 40)
    for vdtype in (np.int32, np.float32):
        v = (datagen.splitmix64(11, n) % np.uint64(100000)).astype(vdtype)
        dk, dv = dev.DeviceArray.from_numpy(k), dev.DeviceArray.from_numpy(v)
        assert np.array_equal(dev.inclusive_scan_by_key(dk, dv, op=op).numpy(),
                              oracle.inclusive_scan_by_key(k, v, op=op))
        assert np.array_equal(dev.exclusive_scan_by_key(dk, dv, init=50000, op=op).numpy(),
                              oracle.exclusive_scan_by_key(k, v, init=50000, op=op))


def test_scan_by_key_segment_shapes(dev, oracle):
    """One long segment, all segments of length one, and a segment border on every tile border."""
    n = 3 * 16384 + 5
    v = (datagen.splitmix64(2, n) % np.uint64(1000)).astype(np.int32)
    for k in (np.zeros(n, np.int32), np.arange(n, dtype=np.int32), (np.arange(n) // 16384).astype(np.int32),
              (np.arange(n) // 64).astype(np.int32)):
        dk, dv = dev.DeviceArray.from_numpy(k), dev.DeviceArray.from_numpy(v)
        assert np.array_equal(dev.inclusive_scan_by_key(dk, dv).numpy(), oracle.inclusive_scan_by_key(k, v))
        assert np.array_equal(dev.exclusive_scan_by_key(dk, dv, init=-3).numpy(),
                              oracle.exclusive_scan_by_key(k, v, init=-3))


def test_inclusive_scan_by_key_in_place(dev, oracle):
    n = (1 << 18) + 9
    k = _keys(n, np.int32, 8, 12)
    v = (datagen.splitmix64(4, n) % np.uint64(1000)).astype(np.int64)
    dk, dv = dev.DeviceArray.from_numpy(k), dev.DeviceArray.from_numpy(v)
    dev.inclusive_scan_by_key(dk, dv, out=dv)
    assert np.array_equal(dv.numpy(), oracle.inclusive_scan_by_key(k, v))


@pytest.mark.parametrize("n", [100, (1 << 18) + 9, (1 << 22) + 5])
def test_exclusive_scan_by_key_in_place(dev, oracle, n):
    # the output on the values themselves, as testing/scan_by_key.cu:463-490 runs it: many tiles, whose first
    # elements continue segments of the tile before them
    k = _keys(n, np.int32, 8, 300)
    v = (datagen.splitmix64(4, n) % np.uint64(1000)).astype(np.int64)
    dk, dv = dev.DeviceArray.from_numpy(k), dev.DeviceArray.from_numpy(v)
    dev.exclusive_scan_by_key(dk, dv, init=7, out=dv)
    assert np.array_equal(dv.numpy(), oracle.exclusive_scan_by_key(k, v, init=7))


def test_scan_by_key_unaligned(dev, oracle):
    n = 50001
    k = _keys(n, np.int32, 6, 9)
    v = (datagen.splitmix64(3, n) % np.uint64(1000)).astype(np.int32)
    dk, dv = dev.DeviceArray.from_numpy(k), dev.DeviceArray.from_numpy(v)
    vk = dev.DeviceArray(n - 1, dk.dtype, dk.storage[4:])
    vv = dev.DeviceArray(n - 1, dv.dtype, dv.storage[4:])
    assert np.array_equal(dev.inclusive_scan_by_key(vk, vv).numpy(), oracle.inclusive_scan_by_key(k[1:], v[1:]))
    assert np.array_equal(dev.exclusive_scan_by_key(vk, vv, init=2).numpy(),
                          oracle.exclusive_scan_by_key(k[1:], v[1:], init=2))


@pytest.mark.parametrize("mean", [1, 8, 1000])
def test_scan_by_key_float_within_tolerance(dev, oracle, mean):
    n = (1 << 21) + 77
    k, v = datagen.c4_segments(n, mean) if mean > 1 else (np.arange(n, dtype=np.int32), datagen.u01(3, n))
    dk, dv = dev.DeviceArray.from_numpy(k), dev.DeviceArray.from_numpy(v)
    head = np.r_[True, k[1:] != k[:-1]]
    starts = np.flatnonzero(head)
    seg_of = np.cumsum(head) - 1
    # float64 reference of the inclusive and exclusive segment sums
    c = np.cumsum(v.astype(np.float64))
    base = np.r_[0.0, c[:-1]][starts][seg_of]
    incl64 = c - base
    excl64 = incl64 - v.astype(np.float64) + 0.25
    got = dev.inclusive_scan_by_key(dk, dv).numpy().astype(np.float64)
    ref = oracle.inclusive_scan_by_key(k, v).astype(np.float64)
    assert np.all(np.abs(got - incl64) <= REL_TOL * np.abs(incl64) + 1e-30)
    assert np.all(np.abs(got - ref) <= 2 * REL_TOL * np.abs(incl64) + 1e-30)
    got = dev.exclusive_scan_by_key(dk, dv, init=0.25).numpy().astype(np.float64)
    ref = oracle.exclusive_scan_by_key(k, v, init=0.25).astype(np.float64)
    assert np.all(np.abs(got - excl64) <= REL_TOL * np.abs(excl64) + 1e-30)
    assert np.all(np.abs(got - ref) <= 2 * REL_TOL * np.abs(excl64) + 1e-30)


@pytest.mark.parametrize("dtype", INT_DTYPES + [np.float32, np.float64])
def test_count_if(dev, oracle, dtype):
    for n in SIZES:
        x = (datagen.splitmix64(21, n) % np.uint64(200)).astype(np.int64) - (0 if np.dtype(dtype).kind == "u" else 100)
        x = x.astype(dtype)
        d = dev.DeviceArray.from_numpy(x)
        for cmp, thr in ((dev.LT, 50), (dev.GE, 0), (dev.EQ, 7), (dev.NE, 7), (dev.NONZERO, 0)):
            got = dev.count_if(d, cmp, thr)
            assert got == oracle.count_if(x, cmp, thr), (dtype, n, cmp)


def test_count_if_unaligned_and_known_answer(dev):
    # testing/count.cu:11-24: {1,1,0,0,1} has three non-zero elements, two equal to zero
    x = np.array([1, 1, 0, 0, 1], np.int32)
    d = dev.DeviceArray.from_numpy(x)
    assert dev.count_if(d, dev.NONZERO) == 3 and dev.count_if(d, dev.EQ, 0) == 2
    big = (datagen.splitmix64(5, 100001) % np.uint64(3)).astype(np.int32)
    d = dev.DeviceArray.from_numpy(big)
    view = dev.DeviceArray(big.size - 1, d.dtype, d.storage[4:])  # 4-byte aligned only
    assert dev.count_if(view, dev.EQ, 1) == int((big[1:] == 1).sum())


@pytest.mark.parametrize("dtype", INT_DTYPES)
def test_inner_product_integers_exact(dev, oracle, dtype):
    for n in SIZES:
        a = (datagen.splitmix64(31, n) >> np.uint64(7)).astype(dtype)
        b = (datagen.splitmix64(32, n) >> np.uint64(9)).astype(dtype)
        da, db = dev.DeviceArray.from_numpy(a), dev.DeviceArray.from_numpy(b)
        got = dev.inner_product(da, db, init=3).numpy()[0]
        assert got == oracle.inner_product(a, b, init=3), (dtype, n)


def test_inner_product_known_answer(dev):
    # testing/inner_product.cu:11-22: (1,-2,3) . (-4,5,6) + 3 = 7
    a, b = np.array([1, -2, 3], np.int32), np.array([-4, 5, 6], np.int32)
    got = dev.inner_product(dev.DeviceArray.from_numpy(a), dev.DeviceArray.from_numpy(b), init=3).numpy()[0]
    assert got == 7


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_inner_product_float_within_tolerance(dev, oracle, dtype):
    n = (1 << 22) + 3
    a = datagen.u01(41, n).astype(dtype)
    b = (datagen.u01(42, n) - 0.25).astype(dtype)
    da, db = dev.DeviceArray.from_numpy(a), dev.DeviceArray.from_numpy(b)
    got = float(dev.inner_product(da, db, init=1.5).numpy()[0])
    exact = float(np.dot(a.astype(np.float64), b.astype(np.float64)) + 1.5)
    tol = REL_TOL if dtype == np.float32 else 1e-12
    assert abs(got - exact) <= tol * abs(exact)
    assert abs(got - float(oracle.inner_product(a, b, init=1.5))) <= 2 * tol * abs(exact)
