"""GPU parity: thrust_amd_reduce / inclusive_scan / exclusive_scan against the CPU oracle.

Mirrors the differential structure of the reference's testing/reduce.cu:80-95 and
testing/scan.cu:365-401 (same algorithm on host and device, results compared), with
the size list of testing/unittest/testframework.cu:21-31 around tile boundaries.
Integer results must be bit-exact; float32 within 1e-5 relative (association order differs).
"""
import numpy as np
import pytest

from thrust_amd import datagen

pytestmark = pytest.mark.gpu

SIZES = [0, 1, 2, 3, 63, 64, 65, 255, 256, 257, 1023, 4095, 4096, 4097, 8191, 8192, 8193,
         65535, 65536, 65537, 100003, (1 << 20) + 7, (1 << 22) - 1]
INT_DTYPES = [np.int8, np.uint8, np.int16, np.uint16, np.int32, np.uint32, np.int64, np.uint64]


def _ints(n, dtype, seed):
    raw = datagen.splitmix64(seed, n)
    return raw.astype(dtype) if np.dtype(dtype).itemsize == 8 else (raw >> np.uint64(17)).astype(dtype)


@pytest.mark.parametrize("dtype", INT_DTYPES)
def test_reduce_plus_int_bit_exact(dev, oracle, dtype):
    for n in SIZES:
        x = _ints(n, dtype, 7)
        d = dev.DeviceArray.from_numpy(x)
        got = dev.reduce(d, dev.PLUS, 3).numpy()[0]
        assert got == oracle.reduce(x, oracle_op(dev.PLUS), 3), (dtype, n)


def oracle_op(op):
    return op  # the codes are shared


@pytest.mark.parametrize("op", [1, 2])
@pytest.mark.parametrize("dtype", [np.int32, np.uint64, np.float32, np.float64])
def test_reduce_min_max(dev, oracle, dtype, op):
    for n in [1, 77, 4096, 100003]:
        x = (_ints(n, np.int32, 9).astype(np.float64) / 7.0).astype(dtype)
        init = x[0]
        d = dev.DeviceArray.from_numpy(x)
        assert dev.reduce(d, op, init).numpy()[0] == oracle.reduce(x, op, init)


def test_reduce_float_sum_tolerance(dev, oracle):
    for n in [1, 1000, 65537, (1 << 22) + 5]:
        x = datagen.u01(11, n)
        d = dev.DeviceArray.from_numpy(x)
        got = float(dev.reduce(d, dev.PLUS, 0).numpy()[0])
        ref64 = float(np.sum(x.astype(np.float64)))
        assert abs(got - ref64) <= 1e-5 * abs(ref64)
        assert abs(got - float(oracle.reduce(x, 0, 0))) <= 1e-5 * abs(ref64)


def test_reduce_unaligned_input(dev, oracle):
    x = _ints(100003, np.int32, 13)
    d = dev.DeviceArray.from_numpy(x)
    for off in [1, 2, 3]:
        view = dev.DeviceArray(x.size - off, d.dtype, d.storage[off * 4:])
        assert dev.reduce(view, dev.PLUS, 0).numpy()[0] == oracle.reduce(x[off:], 0, 0)


@pytest.mark.parametrize("dtype", INT_DTYPES)
def test_scans_int_bit_exact(dev, oracle, dtype):
    for n in SIZES:
        x = _ints(n, dtype, 21)
        d = dev.DeviceArray.from_numpy(x)
        assert np.array_equal(dev.inclusive_scan(d).numpy(), oracle.inclusive_scan(x)), (dtype, n)
        assert np.array_equal(dev.exclusive_scan(d, 5).numpy(), oracle.exclusive_scan(x, 5)), (dtype, n)


def test_scan_in_place_and_unaligned(dev, oracle):
    x = _ints(70001, np.int32, 23)
    d = dev.DeviceArray.from_numpy(x)
    dev.inclusive_scan(d, out=d)
    assert np.array_equal(d.numpy(), oracle.inclusive_scan(x))
    d = dev.DeviceArray.from_numpy(x)
    view = dev.DeviceArray(x.size - 1, d.dtype, d.storage[4:])
    dev.exclusive_scan(view, 9, out=view)
    assert np.array_equal(view.numpy(), oracle.exclusive_scan(x[1:], 9))


@pytest.mark.parametrize("op", [1, 2])
def test_scan_min_max(dev, oracle, op):
    x = _ints(50001, np.int32, 29)
    d = dev.DeviceArray.from_numpy(x)
    assert np.array_equal(dev.inclusive_scan(d, op=op).numpy(), oracle.inclusive_scan(x, op))
    xf = x.astype(np.float32)
    d = dev.DeviceArray.from_numpy(xf)
    assert np.array_equal(dev.inclusive_scan(d, op=op).numpy(), oracle.inclusive_scan(xf, op))


def test_scan_float_tolerance(dev, oracle):
    n = (1 << 20) + 3
    x = datagen.u01(31, n)
    d = dev.DeviceArray.from_numpy(x)
    got = dev.inclusive_scan(d).numpy().astype(np.float64)
    ref64 = np.cumsum(x.astype(np.float64))
    assert np.max(np.abs(got - ref64) / ref64.clip(1e-30)) <= 1e-5
    seq = oracle.inclusive_scan(x).astype(np.float64)
    # the sequential float32 oracle itself drifts; compare both against float64
    assert np.max(np.abs(got - ref64)) <= np.max(np.abs(seq - ref64)) + 1e-5 * ref64[-1]


def test_config1_full_size_closed_form(dev):
    """Config 1 at N=2^28: int32 sum and scan wrap modulo 2^32; checked against numpy int64 mod 2^32."""
    n = 1 << 28
    x = datagen.c1_int32(n)
    d = dev.DeviceArray.from_numpy(x)
    total = int(np.sum(x.astype(np.int64)))
    got = int(dev.reduce(d, dev.PLUS, 0).numpy()[0])
    assert (got - total) % (1 << 32) == 0
    out = dev.inclusive_scan(d).numpy()
    ref = np.cumsum(x.astype(np.int64)).astype(np.uint32).view(np.int32)  # low 32 bits
    assert np.array_equal(out, ref)
