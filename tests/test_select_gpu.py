"""GPU parity: copy_if, partition_copy, stable_partition, unique, unique_by_key against the CPU oracle.

Selection is an order-preserving filter, so every output is compared bit for bit.
Mirrors testing/copy.cu:273-294, testing/partition.cu:688-703, testing/unique.cu and
testing/unique_by_key.cu:257-293 (host result vs device result on the same input).
"""
import numpy as np
import pytest

from thrust_amd import datagen

pytestmark = pytest.mark.gpu

SIZES = [0, 1, 2, 63, 64, 65, 1000, 4097, 16383, 16384, 16385, 32769, 100003, (1 << 20) + 13]
CMPS = list(range(7))


def _vals(n, dtype, seed):
    raw = datagen.splitmix64(seed, n)
    dt = np.dtype(dtype)
    if dt.kind == "f":
        return ((raw >> np.uint64(40)).astype(np.float64) / (1 << 24)).astype(dtype)
    return (raw % np.uint64(200)).astype(dtype)


@pytest.mark.parametrize("dtype", [np.float32, np.int32, np.uint8, np.int16, np.uint64, np.float64])
def test_copy_if_sizes(dev, oracle, dtype):
    thr = 0.5 if np.dtype(dtype).kind == "f" else 100
    for n in SIZES:
        x = _vals(n, dtype, 3)
        d = dev.DeviceArray.from_numpy(x)
        out, cnt = dev.copy_if(d, dev.LT, thr)
        ref = oracle.copy_if(x, dev.LT, thr)
        assert cnt == ref.size and np.array_equal(out.numpy(cnt), ref), (dtype, n)


@pytest.mark.parametrize("cmp", CMPS)
def test_copy_if_predicates(dev, oracle, cmp):
    x = _vals(50001, np.int32, 5)
    d = dev.DeviceArray.from_numpy(x)
    out, cnt = dev.copy_if(d, cmp, 100)
    ref = oracle.copy_if(x, cmp, 100)
    assert cnt == ref.size and np.array_equal(out.numpy(cnt), ref)


def test_copy_if_none_and_all_selected(dev):
    x = _vals(40001, np.float32, 7)
    d = dev.DeviceArray.from_numpy(x)
    out, cnt = dev.copy_if(d, dev.LT, -1.0)
    assert cnt == 0
    out, cnt = dev.copy_if(d, dev.LT, 2.0)
    assert cnt == x.size and np.array_equal(out.numpy(), x)


@pytest.mark.parametrize("item", [np.uint8, np.uint16, np.float32, np.uint64])
@pytest.mark.parametrize("sdtype", [np.int32, np.uint8, np.float32])
def test_copy_if_stencil(dev, oracle, item, sdtype):
    for n in [0, 1, 777, 16385, 70001]:
        x = _vals(n, item, 9)
        st = _vals(n, sdtype, 11)
        thr = 0.5 if np.dtype(sdtype).kind == "f" else 100
        d, ds = dev.DeviceArray.from_numpy(x), dev.DeviceArray.from_numpy(st)
        out, cnt = dev.copy_if(d, dev.GE, thr, stencil=ds)
        ref = oracle.copy_if(x, dev.GE, thr, stencil=st)
        assert cnt == ref.size and np.array_equal(out.numpy(cnt), ref), (item, sdtype, n)
        # default stencil predicate: "is true"
        out, cnt = dev.copy_if(d, dev.NONZERO, 0, stencil=ds)
        ref = oracle.copy_if(x, dev.NONZERO, 0, stencil=st)
        assert cnt == ref.size and np.array_equal(out.numpy(cnt), ref)


@pytest.mark.parametrize("sdtype", [np.int8, np.uint8, np.int16, np.uint16, np.int32, np.uint32, np.int64, np.uint64,
                                    np.float32, np.float64])
def test_stencil_forms_for_every_stencil_type_and_item_width(dev, oracle, sdtype):
    """copy_if and partition_copy by stencil run one kernel per (stencil type, item width, one or two
    outputs): each of them once, on a ragged size of several tiles, with every comparison code."""
    n = 100003
    st = _vals(n, sdtype, 23)
    ds = dev.DeviceArray.from_numpy(st)
    thr = 0.5 if np.dtype(sdtype).kind == "f" else 100
    for item in (np.uint8, np.uint16, np.uint32, np.uint64):
        x = _vals(n, item, 29)
        d = dev.DeviceArray.from_numpy(x)
        for cmp in (dev.LT, dev.LE, dev.GT, dev.GE, dev.EQ, dev.NE, dev.NONZERO):
            out, cnt = dev.copy_if(d, cmp, thr, stencil=ds)
            ref = oracle.copy_if(x, cmp, thr, stencil=st)
            assert cnt == ref.size and np.array_equal(out.numpy(cnt), ref), (sdtype, item, cmp)
        ot, of, cnt = dev.partition_copy(d, dev.LT, thr, stencil=ds)
        rt, rf = oracle.partition_copy(x, dev.LT, thr, stencil=st)
        assert cnt == rt.size and np.array_equal(ot.numpy(cnt), rt) and np.array_equal(of.numpy(n - cnt), rf), (sdtype, item)


@pytest.mark.parametrize("dtype", [np.float32, np.uint8, np.uint64])
def test_copy_if_in_place(dev, oracle, dtype):
    """out aliases in, the form remove_if uses (thrust/system/cuda/detail/remove.h:54-66): a
    tile is written only after every earlier tile has been read."""
    thr = 0.5 if np.dtype(dtype).kind == "f" else 100
    for n in [1, 777, 16384, 16385, 70001, (1 << 22) + 11]:
        x = _vals(n, dtype, 17)
        for cmp in (dev.GE, dev.LT):
            d = dev.DeviceArray.from_numpy(x)
            _, cnt = dev.copy_if(d, cmp, thr, out=d)
            ref = oracle.copy_if(x, cmp, thr)
            assert cnt == ref.size and np.array_equal(d.numpy()[:cnt], ref), (dtype, n, cmp)
        st = _vals(n, np.int32, 19)
        d, ds = dev.DeviceArray.from_numpy(x), dev.DeviceArray.from_numpy(st)
        _, cnt = dev.copy_if(d, dev.EQ, 0, stencil=ds, out=d)
        ref = oracle.copy_if(x, dev.EQ, 0, stencil=st)
        assert cnt == ref.size and np.array_equal(d.numpy()[:cnt], ref), (dtype, n, "stencil")


def test_copy_if_unaligned(dev, oracle):
    x = _vals(40003, np.float32, 13)
    d = dev.DeviceArray.from_numpy(x)
    view = dev.DeviceArray(x.size - 3, d.dtype, d.storage[12:])
    out, cnt = dev.copy_if(view, dev.LT, 0.5)
    ref = oracle.copy_if(x[3:], dev.LT, 0.5)
    assert cnt == ref.size and np.array_equal(out.numpy(cnt), ref)


@pytest.mark.parametrize("dtype", [np.float32, np.int32, np.uint8, np.uint64])
def test_partition_copy_and_in_place(dev, oracle, dtype):
    thr = 0.5 if np.dtype(dtype).kind == "f" else 100
    for n in SIZES:
        x = _vals(n, dtype, 15)
        d = dev.DeviceArray.from_numpy(x)
        ot, of, cnt = dev.partition_copy(d, dev.LT, thr)
        rt, rf = oracle.partition_copy(x, dev.LT, thr)
        assert cnt == rt.size
        assert np.array_equal(ot.numpy(cnt), rt) and np.array_equal(of.numpy(n - cnt), rf), (dtype, n)
        cnt2 = dev.stable_partition(d, dev.LT, thr)
        ref, rcnt = oracle.stable_partition(x, dev.LT, thr)
        assert cnt2 == rcnt and np.array_equal(d.numpy(), ref), (dtype, n)


def test_stable_partition_stencil(dev, oracle):
    for n in [1, 999, 16385, 65537]:
        x = _vals(n, np.float64, 17)
        st = _vals(n, np.int32, 19)
        d, ds = dev.DeviceArray.from_numpy(x), dev.DeviceArray.from_numpy(st)
        cnt = dev.stable_partition(d, dev.LT, 50, stencil=ds)
        ref, rcnt = oracle.stable_partition(x, dev.LT, 50, stencil=st)
        assert cnt == rcnt and np.array_equal(d.numpy(), ref)


@pytest.mark.parametrize("sdtype", [np.uint8, np.uint16, np.int32, np.float32, np.uint64, np.float64])
def test_stable_partition_stencil_in_place_one_pass(dev, oracle, sdtype):
    """The in-place form tests the stencil in its own type with the items as payload (no flag array): every item width,
    selectivities that make the sweep run from either end, sizes of many tiles with a ragged last one."""
    for item in (np.uint8, np.int16, np.float32, np.int64):
        for n, thr in ((70001, 10), ((1 << 21) + 77, 150), ((1 << 21) + 77, 100)):
            x = _vals(n, item, 23)
            st = _vals(n, sdtype, 29)
            d, ds = dev.DeviceArray.from_numpy(x), dev.DeviceArray.from_numpy(st)
            cnt = dev.stable_partition(d, dev.LT, thr, stencil=ds)
            ref, rcnt = oracle.stable_partition(x, dev.LT, thr, stencil=st)
            assert cnt == rcnt and np.array_equal(d.numpy(), ref), (sdtype, item, n, thr)
            assert np.array_equal(ds.numpy(), st)  # the stencil is only read


def test_config5_full_size(dev):
    """Config 5 at N=2^28 float32, t = 0.5 and 0.05: compared with numpy's boolean filter
    (the definition of an order-preserving selection)."""
    n = 1 << 28
    x = datagen.c5_float32(n)
    d = dev.DeviceArray.from_numpy(x)
    for t in (0.5, 0.05):
        out, cnt = dev.copy_if(d, dev.LT, t)
        mask = x < np.float32(t)
        assert cnt == int(mask.sum())
        assert np.array_equal(out.numpy(cnt), x[mask])
        work = d.clone()
        cnt = dev.stable_partition(work, dev.LT, t)
        got = work.numpy()
        assert cnt == int(mask.sum())
        assert np.array_equal(got[:cnt], x[mask]) and np.array_equal(got[cnt:], x[~mask])


def _runs(n, dtype, seed, mean):
    lens = (datagen.splitmix64(seed, n) % np.uint64(2 * mean)).astype(np.int64) + 1
    ids = np.repeat(np.arange(n, dtype=np.int64), lens)[:n]
    dt = np.dtype(dtype)
    vals = (datagen.splitmix64(seed + 1, n) % np.uint64(97)).astype(np.int64)
    keys = vals[ids]  # equal neighbours inside a run, possibly across runs too
    return keys.astype(dtype)


@pytest.mark.parametrize("dtype", [np.int32, np.uint8, np.int64, np.float32, np.uint16, np.float64])
def test_unique_sizes(dev, oracle, dtype):
    for n in SIZES:
        x = _runs(n, dtype, 21, 3)
        d = dev.DeviceArray.from_numpy(x)
        out, cnt = dev.unique(d)
        ref = oracle.unique(x)
        assert cnt == ref.size and np.array_equal(out.numpy(cnt), ref), (dtype, n)
        # in place: out aliases in
        _, cnt2 = dev.unique(d, out=d)
        assert cnt2 == ref.size and np.array_equal(d.numpy(cnt2), ref), (dtype, n)


@pytest.mark.parametrize("kdtype", [np.int32, np.uint64, np.float32, np.uint8])
@pytest.mark.parametrize("vdtype", [np.uint8, np.uint16, np.float32, np.uint64])
def test_unique_by_key(dev, oracle, kdtype, vdtype):
    for n in [0, 1, 2, 1000, 16385, 100003]:
        k = _runs(n, kdtype, 23, 4)
        v = np.arange(n).astype(vdtype)
        dk, dv = dev.DeviceArray.from_numpy(k), dev.DeviceArray.from_numpy(v)
        ko, vo, cnt = dev.unique_by_key(dk, dv)
        rk, rv = oracle.unique_by_key(k, v)
        assert cnt == rk.size
        assert np.array_equal(ko.numpy(cnt), rk) and np.array_equal(vo.numpy(cnt), rv), (kdtype, vdtype, n)
        _, _, cnt2 = dev.unique_by_key(dk, dv, keys_out=dk, values_out=dv)
        assert cnt2 == rk.size
        assert np.array_equal(dk.numpy(cnt2), rk) and np.array_equal(dv.numpy(cnt2), rv)


def test_unique_float_nan_and_zero(dev, oracle):
    x = np.array([0.0, -0.0, 0.0, np.nan, np.nan, 1.0, 1.0, -0.0], np.float32)
    d = dev.DeviceArray.from_numpy(x)
    out, cnt = dev.unique(d)
    ref = oracle.unique(x)
    assert cnt == ref.size
    assert np.array_equal(out.numpy(cnt).view(np.uint32), ref.view(np.uint32))
