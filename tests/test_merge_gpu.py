"""GPU parity: thrust_amd_merge / thrust_amd_merge_by_key against the CPU oracle.

A stable merge with the "range A first on ties" rule has a unique answer including the
values, so everything is compared bit for bit (testing/merge.cu:11-38,
testing/merge_by_key.cu:10-45,129- are the models).
"""
import numpy as np
import pytest

from thrust_amd import datagen

pytestmark = pytest.mark.gpu

SIZE_PAIRS = [(0, 0), (0, 5), (5, 0), (1, 1), (3, 4), (100, 1), (1, 100), (4096, 4096), (4095, 4097),
              (5000, 7000), (100003, 3), (3, 100003), (70001, 90001), ((1 << 20) + 3, (1 << 19) + 7)]


def _sorted(n, dtype, seed, modulus=1000, descending=False):
    raw = datagen.splitmix64(seed, n) % np.uint64(modulus)
    x = np.sort(raw.astype(np.int64) - (modulus // 2 if np.dtype(dtype).kind in "if" else 0)).astype(dtype)
    return x[::-1].copy() if descending else x


@pytest.mark.parametrize("dtype", [np.int32, np.uint32, np.uint8, np.int16, np.int64, np.uint64, np.float32, np.float64])
def test_merge_keys(dev, oracle, dtype):
    mod = 200 if np.dtype(dtype).itemsize == 1 else 1000
    for na, nb in SIZE_PAIRS:
        a, b = _sorted(na, dtype, 3, mod), _sorted(nb, dtype, 5, mod)
        da, db = dev.DeviceArray.from_numpy(a), dev.DeviceArray.from_numpy(b)
        out = dev.merge(da, db)
        assert np.array_equal(out.numpy(), oracle.merge(a, b)), (dtype, na, nb)


@pytest.mark.parametrize("kdtype", [np.uint32, np.int32, np.float32, np.uint64])
@pytest.mark.parametrize("vdtype", [np.uint8, np.uint16, np.uint32, np.uint64])
def test_merge_by_key_ties_take_first_range(dev, oracle, kdtype, vdtype):
    for na, nb in SIZE_PAIRS:
        ka, kb = _sorted(na, kdtype, 7, 50), _sorted(nb, kdtype, 9, 50)  # many ties
        va = (np.arange(na) % 251).astype(vdtype)
        vb = ((np.arange(nb) % 251) + 1).astype(vdtype)
        out_k, out_v = dev.merge_by_key(*(dev.DeviceArray.from_numpy(x) for x in (ka, kb, va, vb)))
        rk, rv = oracle.merge_by_key(ka, kb, va, vb)
        assert np.array_equal(out_k.numpy(), rk) and np.array_equal(out_v.numpy(), rv), (kdtype, vdtype, na, nb)


def test_merge_descending(dev, oracle):
    for na, nb in [(1000, 3000), (70001, 5)]:
        ka, kb = _sorted(na, np.int32, 11, 300, True), _sorted(nb, np.int32, 13, 300, True)
        va, vb = np.arange(na, dtype=np.uint32), np.arange(nb, dtype=np.uint32) + 10 ** 6
        out_k, out_v = dev.merge_by_key(*(dev.DeviceArray.from_numpy(x) for x in (ka, kb, va, vb)),
                                        descending=True)
        rk, rv = oracle.merge_by_key(ka, kb, va, vb, descending=True)
        assert np.array_equal(out_k.numpy(), rk) and np.array_equal(out_v.numpy(), rv)
        out = dev.merge(dev.DeviceArray.from_numpy(ka), dev.DeviceArray.from_numpy(kb), descending=True)
        assert np.array_equal(out.numpy(), oracle.merge(ka, kb, descending=True))


def test_merge_float_signed_zero_ties(dev, oracle):
    a = np.array([-1.0, 0.0, 0.0, 2.0], np.float32)
    b = np.array([-0.0, -0.0, 0.0, 3.0], np.float32)
    out = dev.merge(dev.DeviceArray.from_numpy(a), dev.DeviceArray.from_numpy(b))
    assert np.array_equal(out.numpy().view(np.uint32), oracle.merge(a, b).view(np.uint32))


def test_one_range_entirely_before_the_other(dev, oracle):
    a = np.arange(50000, dtype=np.uint32)
    b = np.arange(50000, 120001, dtype=np.uint32)
    for x, y in ((a, b), (b, a)):
        out = dev.merge(dev.DeviceArray.from_numpy(x), dev.DeviceArray.from_numpy(y))
        assert np.array_equal(out.numpy(), oracle.merge(x, y))


def test_config5_merge_full_size(dev):
    """Config 5: two independently sorted 2^27 uint32 arrays with uint32 payloads.  Checked
    against numpy: a stable sort of the concatenation A|B by key is exactly the merge with
    A first on ties."""
    n = 1 << 27
    (ka, va), (kb, vb) = datagen.c5_merge_inputs(n)
    out_k, out_v = dev.merge_by_key(*(dev.DeviceArray.from_numpy(x) for x in (ka, kb, va, vb)))
    keys = np.concatenate([ka, kb])
    vals = np.concatenate([va, vb])
    order = np.argsort(keys, kind="stable")
    assert np.array_equal(out_k.numpy(), keys[order])
    assert np.array_equal(out_v.numpy(), vals[order])
