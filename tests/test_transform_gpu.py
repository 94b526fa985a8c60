"""GPU parity: thrust_amd_transform_reduce, thrust_amd_transform_inclusive_scan and
thrust_amd_transform_exclusive_scan against the CPU oracle.

Integer results are exact for every association order; float32 results are compared with
the oracle within 1e-5 relative and with a float64 evaluation.  Models:
testing/transform_reduce.cu:70-100 (negate + plus, init), testing/transform_scan.cu:140-300
(negate + plus, init, in place) and :355-399 (identity + maximum).
"""
import numpy as np
import pytest

from thrust_amd import datagen

pytestmark = pytest.mark.gpu

SIZES = [0, 1, 2, 63, 64, 65, 1000, 4095, 4096, 4097, 49151, 49152, 49153, 100003, (1 << 20) + 13, (1 << 23) + 5]
REL_TOL = 1e-5
INT_DTYPES = [np.int8, np.uint8, np.int16, np.uint16, np.int32, np.uint32, np.int64, np.uint64]
IDENTITY, NEGATE, SQUARE = range(3)


def _ints(n, dtype, seed):
    x = (datagen.splitmix64(seed, n) % np.uint64(2001)).astype(np.int64) - 1000
    return x.astype(dtype)


@pytest.mark.parametrize("dtype", INT_DTYPES)
@pytest.mark.parametrize("unary", [IDENTITY, NEGATE, SQUARE])
def test_transform_reduce_integers_exact(dev, oracle, dtype, unary):
    for n in SIZES:
        x = _ints(n, dtype, 51)
        d = dev.DeviceArray.from_numpy(x)
        for op in (dev.PLUS, dev.MIN, dev.MAX):
            got = dev.transform_reduce(d, unary, op=op, init=3).numpy()[0]
            assert got == oracle.transform_reduce(x, unary, op, 3), (dtype, unary, op, n)


@pytest.mark.parametrize("dtype", INT_DTYPES)
@pytest.mark.parametrize("unary", [IDENTITY, NEGATE, SQUARE])
def test_transform_scans_integers_exact(dev, oracle, dtype, unary):
    for n in SIZES:
        x = _ints(n, dtype, 52)
        d = dev.DeviceArray.from_numpy(x)
        for op in (dev.PLUS, dev.MAX):
            got = dev.transform_inclusive_scan(d, unary, op=op).numpy()
            assert np.array_equal(got, oracle.transform_inclusive_scan(x, unary, op)), ("inclusive", dtype, unary, op, n)
            got = dev.transform_exclusive_scan(d, unary, init=11, op=op).numpy()
            assert np.array_equal(got, oracle.transform_exclusive_scan(x, unary, 11, op)), ("exclusive", dtype, unary, op, n)


def test_transform_known_answers(dev):
    # testing/transform_reduce.cu:70-83 and testing/transform_scan.cu:152-175
    x = dev.DeviceArray.from_numpy(np.array([1, -2, 3], np.int32))
    assert dev.transform_reduce(x, NEGATE, init=10).numpy()[0] == 8
    x = dev.DeviceArray.from_numpy(np.array([1, 3, -2, 4, -5], np.int32))
    assert dev.transform_inclusive_scan(x, NEGATE).numpy().tolist() == [-1, -4, -2, -6, -1]
    assert dev.transform_exclusive_scan(x, NEGATE, init=0).numpy().tolist() == [0, -1, -4, -2, -6]
    assert dev.transform_exclusive_scan(x, NEGATE, init=3).numpy().tolist() == [3, 2, -1, 1, -3]
    # testing/transform_scan.cu:355-399
    x = dev.DeviceArray.from_numpy(np.array([5, 0, 5, 8, 6, 7, 5, 3, 0, 9], np.int32))
    assert dev.transform_inclusive_scan(x, IDENTITY, op=dev.MAX).numpy().tolist() == [5, 5, 5, 8, 8, 8, 8, 8, 8, 9]
    assert dev.transform_exclusive_scan(x, IDENTITY, init=0, op=dev.MAX).numpy().tolist() == [0, 5, 5, 5, 8, 8, 8, 8, 8, 8]


def test_transform_scans_in_place_and_unaligned(dev, oracle):
    n = (1 << 18) + 9
    x = _ints(n, np.int32, 53)
    d = dev.DeviceArray.from_numpy(x)
    dev.transform_inclusive_scan(d, NEGATE, out=d)
    assert np.array_equal(d.numpy(), oracle.transform_inclusive_scan(x, NEGATE))
    d = dev.DeviceArray.from_numpy(x)
    dev.transform_exclusive_scan(d, SQUARE, init=7, out=d)
    assert np.array_equal(d.numpy(), oracle.transform_exclusive_scan(x, SQUARE, 7))
    d = dev.DeviceArray.from_numpy(x)
    view = dev.DeviceArray(n - 1, d.dtype, d.storage[4:])  # 4-byte aligned only
    assert np.array_equal(dev.transform_inclusive_scan(view, SQUARE).numpy(), oracle.transform_inclusive_scan(x[1:], SQUARE))
    assert dev.transform_reduce(view, SQUARE, init=1).numpy()[0] == oracle.transform_reduce(x[1:], SQUARE, init=1)


def test_int_min_negates_to_itself_and_squares_wrap(dev, oracle):
    x = np.array([np.iinfo(np.int32).min, 65536, -65536, 46341, -1], np.int32)
    d = dev.DeviceArray.from_numpy(x)
    for unary in (NEGATE, SQUARE):
        assert np.array_equal(dev.transform_inclusive_scan(d, unary).numpy(), oracle.transform_inclusive_scan(x, unary))
        assert dev.transform_reduce(d, unary, op=dev.MIN, init=0).numpy()[0] == oracle.transform_reduce(x, unary, dev.MIN, 0)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_transform_float_within_tolerance(dev, oracle, dtype):
    n = (1 << 22) + 3
    x = (datagen.u01(61, n) - 0.25).astype(dtype)
    d = dev.DeviceArray.from_numpy(x)
    tol = REL_TOL if dtype == np.float32 else 1e-11  # numpy's own float64 running sum is the yardstick there
    x64 = x.astype(np.float64)
    exact = float(np.sum(x64 * x64) + 1.5)
    got = float(dev.transform_reduce(d, SQUARE, init=1.5).numpy()[0])
    assert abs(got - exact) <= tol * abs(exact)
    # the reference's own chunked left fold drifts from the exact sum; allow it that much
    ref = float(oracle.transform_reduce(x, SQUARE, init=1.5))
    assert abs(got - ref) <= abs(ref - exact) + tol * abs(exact)
    # scans of squares: every prefix is a sum of non-negative terms
    sq64 = (x * x).astype(np.float64)  # the squares as the kernel rounds them
    exact_scan = np.cumsum(sq64)
    got = dev.transform_inclusive_scan(d, SQUARE).numpy().astype(np.float64)
    assert np.all(np.abs(got - exact_scan) <= tol * exact_scan + 1e-30)
    seq = oracle.transform_inclusive_scan(x, SQUARE).astype(np.float64)
    assert np.max(np.abs(got - exact_scan)) <= np.max(np.abs(seq - exact_scan)) + tol * exact_scan[-1]
    got = dev.transform_exclusive_scan(d, SQUARE, init=0.5).numpy().astype(np.float64)
    assert np.all(np.abs(got - (exact_scan - sq64 + 0.5)) <= 2 * tol * (exact_scan + 0.5))
    # minimum / maximum of the negated values are exact
    assert dev.transform_reduce(d, NEGATE, op=dev.MAX, init=-9.0).numpy()[0] == np.max(-x)
    assert np.array_equal(dev.transform_inclusive_scan(d, NEGATE, op=dev.MIN).numpy(), np.minimum.accumulate(-x))


def test_transform_rejects_unknown_codes(dev):
    d = dev.DeviceArray.from_numpy(np.zeros(10, np.int32))
    with pytest.raises(dev.ThrustAmdError):
        dev.transform_reduce(d, 3)
    with pytest.raises(dev.ThrustAmdError):
        dev.transform_inclusive_scan(d, -1)
