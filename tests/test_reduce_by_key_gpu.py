"""GPU parity: thrust_amd_reduce_by_key against the CPU oracle.

Keys and run counts are exact; integer folds are exact (wrap-around addition is
associative); float32 sums are compared with the oracle's strict left fold within 1e-5
relative and with a float64 fold (testing/reduce_by_key.cu:115-156 is the model:
host result vs device result on run-heavy keys).
"""
import numpy as np
import pytest

from thrust_amd import datagen

pytestmark = pytest.mark.gpu

SIZES = [0, 1, 2, 63, 64, 65, 1000, 16383, 16384, 16385, 32769, 100003, (1 << 20) + 13]
REL_TOL = 1e-5


def _keys(n, dtype, seed, mean):
    lens = (datagen.splitmix64(seed, n) % np.uint64(2 * mean)).astype(np.int64) + 1
    ids = np.repeat(np.arange(n, dtype=np.int64), lens)[:n]
    vals = (datagen.splitmix64(seed + 1, n) % np.uint64(97)).astype(np.int64)
    return vals[ids].astype(dtype)


@pytest.mark.parametrize("kdtype", [np.int32, np.uint8, np.int64, np.uint16, np.float32, np.float64])
@pytest.mark.parametrize("vdtype", [np.int32, np.uint64, np.int8, np.int16])
def test_integer_values_exact(dev, oracle, kdtype, vdtype):
    for n in SIZES:
        k = _keys(n, kdtype, 3, 5)
        v = (datagen.splitmix64(9, n) >> np.uint64(20)).astype(vdtype)
        dk, dv = dev.DeviceArray.from_numpy(k), dev.DeviceArray.from_numpy(v)
        ko, vo, runs = dev.reduce_by_key(dk, dv)
        rk, rv = oracle.reduce_by_key(k, v)
        assert runs == rk.size, (kdtype, vdtype, n)
        assert np.array_equal(ko.numpy(runs), rk) and np.array_equal(vo.numpy(runs), rv), (kdtype, vdtype, n)


@pytest.mark.parametrize("op", [1, 2])
def test_min_max(dev, oracle, op):
    n = 70001
    k = _keys(n, np.int32, 5, 40)
    for vdtype in (np.int32, np.float32):
        v = (datagen.splitmix64(11, n) % np.uint64(100000)).astype(vdtype)
        dk, dv = dev.DeviceArray.from_numpy(k), dev.DeviceArray.from_numpy(v)
        ko, vo, runs = dev.reduce_by_key(dk, dv, op=op)
        rk, rv = oracle.reduce_by_key(k, v, op=op)
        assert runs == rk.size and np.array_equal(ko.numpy(runs), rk) and np.array_equal(vo.numpy(runs), rv)


@pytest.mark.parametrize("mean", [1, 8, 1000, 100000])
def test_float_sums_within_tolerance(dev, oracle, mean):
    n = (1 << 21) + 77
    k, v = datagen.c4_segments(n, mean) if mean > 1 else (np.arange(n, dtype=np.int32), datagen.u01(3, n))
    dk, dv = dev.DeviceArray.from_numpy(k), dev.DeviceArray.from_numpy(v)
    ko, vo, runs = dev.reduce_by_key(dk, dv)
    rk, rv = oracle.reduce_by_key(k, v)
    assert runs == rk.size and np.array_equal(ko.numpy(runs), rk)
    got = vo.numpy(runs).astype(np.float64)
    starts = np.flatnonzero(np.r_[True, k[1:] != k[:-1]])
    ref64 = np.add.reduceat(v.astype(np.float64), starts)
    assert np.max(np.abs(got - ref64) / np.abs(ref64)) <= REL_TOL
    # The oracle folds strictly left to right in float32 and drifts from the exact sum by
    # itself on long runs (about 1e-5 relative at 1e5 elements): the device may differ from
    # it by that drift plus the tolerance, and by the tolerance alone at the configs' lengths.
    seq = rv.astype(np.float64)
    drift = np.abs(seq - ref64) / np.abs(ref64)
    assert np.all(np.abs(got - seq) / np.abs(ref64) <= drift + REL_TOL)
    if mean <= 1000:
        assert np.max(np.abs(got - seq) / np.abs(ref64)) <= REL_TOL


def test_one_long_run_and_all_distinct(dev, oracle):
    n = 200001
    v = np.ones(n, np.int32)
    for k in (np.zeros(n, np.int32), np.arange(n, dtype=np.int32)):
        dk, dv = dev.DeviceArray.from_numpy(k), dev.DeviceArray.from_numpy(v)
        ko, vo, runs = dev.reduce_by_key(dk, dv)
        rk, rv = oracle.reduce_by_key(k, v)
        assert runs == rk.size and np.array_equal(ko.numpy(runs), rk) and np.array_equal(vo.numpy(runs), rv)


def test_first_key_of_run_is_kept_bitwise(dev, oracle):
    # -0.0 == +0.0 under equal_to: one run, and the reference emits its FIRST key
    k = np.array([-0.0, 0.0, 0.0, 1.0, 1.0, 0.0, -0.0], np.float32)
    v = np.arange(k.size, dtype=np.int32)
    dk, dv = dev.DeviceArray.from_numpy(k), dev.DeviceArray.from_numpy(v)
    ko, vo, runs = dev.reduce_by_key(dk, dv)
    rk, rv = oracle.reduce_by_key(k, v)
    assert runs == rk.size == 3
    assert np.array_equal(ko.numpy(runs).view(np.uint32), rk.view(np.uint32))
    assert np.array_equal(vo.numpy(runs), rv)


def test_unaligned_inputs(dev, oracle):
    n = 50003
    k = _keys(n, np.int32, 13, 6)
    v = (datagen.splitmix64(15, n) >> np.uint64(40)).astype(np.int32)
    dk, dv = dev.DeviceArray.from_numpy(k), dev.DeviceArray.from_numpy(v)
    vk = dev.DeviceArray(n - 1, dk.dtype, dk.storage[4:])
    vv = dev.DeviceArray(n - 1, dv.dtype, dv.storage[4:])
    ko, vo, runs = dev.reduce_by_key(vk, vv)
    rk, rv = oracle.reduce_by_key(k[1:], v[1:])
    assert runs == rk.size and np.array_equal(ko.numpy(runs), rk) and np.array_equal(vo.numpy(runs), rv)


@pytest.mark.parametrize("mean", [8, 1000])
def test_config4_full_size(dev, mean):
    """Config 4 at N=2^28: run count and keys exact; float32 sums against a float64 fold
    within 1e-5 relative; unique_by_key keeps the first value of each run."""
    n = 1 << 28
    k, v = datagen.c4_segments(n, mean)
    dk, dv = dev.DeviceArray.from_numpy(k), dev.DeviceArray.from_numpy(v)
    ko, vo, runs = dev.reduce_by_key(dk, dv)
    starts = np.flatnonzero(np.r_[True, k[1:] != k[:-1]])
    assert runs == starts.size
    assert np.array_equal(ko.numpy(runs), k[starts])
    ref64 = np.add.reduceat(v.astype(np.float64), starts)
    got = vo.numpy(runs).astype(np.float64)
    assert np.max(np.abs(got - ref64) / ref64.clip(1e-30)) <= REL_TOL
    ko, vo, cnt = dev.unique_by_key(dk, dv)
    assert cnt == starts.size
    assert np.array_equal(ko.numpy(cnt), k[starts]) and np.array_equal(vo.numpy(cnt), v[starts])
