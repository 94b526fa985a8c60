"""GPU parity: thrust_amd_merge_sort_keys / thrust_amd_merge_sort_pairs (the stable
comparison sort) against the CPU oracle's restatement of the reference's merge sort.

A stable sort has exactly one right answer, so every comparison is bit-exact.  Sizes sit
on both sides of the lane (16), tile (4096) and run-pair borders, including odd numbers
of tiles, where the last run of a pass has no partner.  Models: testing/stable_sort.cu:
49-110 and testing/stable_sort_by_key.cu:50-125 (equivalent keys keep their input order).
"""
import numpy as np
import pytest

from thrust_amd import datagen

pytestmark = pytest.mark.gpu

SIZES = [0, 1, 2, 15, 16, 17, 255, 256, 257, 4095, 4096, 4097, 8191, 8192, 8193, 3 * 4096 + 5, 5 * 4096,
         100003, (1 << 20) + 13, 5 * (1 << 20) + 7]
DTYPES = [np.int8, np.uint8, np.int16, np.uint16, np.int32, np.uint32, np.int64, np.uint64, np.float32, np.float64]


def _keys(n, dtype, seed, spread):
    raw = (datagen.splitmix64(seed, n) % np.uint64(spread)).astype(np.int64)
    if np.dtype(dtype).kind == "f":
        x = (raw - spread // 2).astype(dtype) / 4
        x[datagen.splitmix64(seed + 1, n) % np.uint64(11) == 0] = -0.0  # equivalent to +0.0, different bits
        return x
    if np.dtype(dtype).kind == "i":
        raw = raw - spread // 2
    return raw.astype(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_merge_sort_keys(dev, oracle, dtype):
    for n in SIZES:
        for descending in (False, True):
            x = _keys(n, dtype, 81 + n % 7, 200)
            d = dev.DeviceArray.from_numpy(x)
            dev.merge_sort_keys(d, descending)
            want = oracle.comparison_sort(x, None, 1 if descending else 0)
            assert d.numpy().tobytes() == want.tobytes(), (dtype, n, descending)


@pytest.mark.parametrize("dtype", [np.int8, np.uint16, np.int32, np.uint64, np.float32, np.float64])
@pytest.mark.parametrize("vdtype", [np.uint8, np.uint16, np.uint32, np.uint64])
def test_merge_sort_pairs_are_stable(dev, oracle, dtype, vdtype):
    for n in SIZES:
        if n > np.iinfo(vdtype).max + 1 and np.dtype(vdtype).itemsize < 4:
            v = (np.arange(n, dtype=np.uint64) * np.uint64(2654435761)).astype(vdtype)  # wraps: still a payload
        else:
            v = np.arange(n, dtype=np.uint64).astype(vdtype)
        for descending in (False, True):
            x = _keys(n, dtype, 91, 37)  # few distinct keys: long runs of equivalents
            dk, dv = dev.DeviceArray.from_numpy(x), dev.DeviceArray.from_numpy(v)
            dev.merge_sort_pairs(dk, dv, descending)
            wk, wv = oracle.comparison_sort(x, v, 1 if descending else 0)
            assert dk.numpy().tobytes() == wk.tobytes(), (dtype, vdtype, n, descending)
            assert np.array_equal(dv.numpy(), wv), (dtype, vdtype, n, descending)


def test_merge_sort_orders_and_special_inputs(dev, oracle):
    n = 3 * 4096 + 77
    v = np.arange(n, dtype=np.uint32)
    cases = {
        "sorted": np.arange(n, dtype=np.int32),
        "reversed": np.arange(n, dtype=np.int32)[::-1].copy(),
        "all equal": np.full(n, 7, np.int32),
        "two values": (np.arange(n) % 2).astype(np.int32),
        "sawtooth": (np.arange(n) % 4099).astype(np.int32),
        "extremes": np.where(np.arange(n) % 3 == 0, np.iinfo(np.int32).min, np.iinfo(np.int32).max).astype(np.int32),
    }
    for name, x in cases.items():
        for descending in (False, True):
            dk, dv = dev.DeviceArray.from_numpy(x), dev.DeviceArray.from_numpy(v)
            dev.merge_sort_pairs(dk, dv, descending)
            wk, wv = oracle.comparison_sort(x, v, 1 if descending else 0)
            assert np.array_equal(dk.numpy(), wk) and np.array_equal(dv.numpy(), wv), (name, descending)


def test_merge_sort_equals_radix_sort_on_integers(dev):
    # two independent implementations of the same unique answer
    n = (1 << 22) + 4099
    x = datagen.splitmix64(5, n).astype(np.uint32)
    v = np.arange(n, dtype=np.uint32)
    a, av = dev.DeviceArray.from_numpy(x), dev.DeviceArray.from_numpy(v)
    b, bv = dev.DeviceArray.from_numpy(x), dev.DeviceArray.from_numpy(v)
    dev.merge_sort_pairs(a, av)
    dev.sort_pairs(b, bv)
    assert np.array_equal(a.numpy(), b.numpy()) and np.array_equal(av.numpy(), bv.numpy())
    s = a.numpy()
    assert np.all(s[:-1] <= s[1:]) and np.array_equal(np.sort(av.numpy()), v)


def test_merge_sort_float_zeros_keep_input_order(dev):
    z = np.array([0.0, -0.0, 1.0, -0.0, 0.0, -1.0], np.float32)
    d = dev.DeviceArray.from_numpy(z)
    dev.merge_sort_keys(d)
    assert d.numpy().tobytes() == np.array([-1.0, 0.0, -0.0, -0.0, 0.0, 1.0], np.float32).tobytes()
    r = dev.DeviceArray.from_numpy(z)
    dev.sort_keys(r)  # the radix path orders by bit pattern: -0.0 first
    assert r.numpy().tobytes() == np.array([-1.0, -0.0, -0.0, 0.0, 0.0, 1.0], np.float32).tobytes()


def test_merge_sort_temp_and_arguments(dev):
    lib = dev.load()
    import ctypes
    need = ctypes.c_size_t(0)
    i32 = dev.DTYPE_OF_NP[np.dtype(np.int32)]
    assert lib.thrust_amd_merge_sort_keys(None, ctypes.byref(need), None, 1 << 20, i32, 0, dev.stream_ptr()) == 0
    assert need.value >= (1 << 20) * 4
    small = ctypes.c_size_t(16)
    d = dev.DeviceArray(1 << 20, i32)
    assert lib.thrust_amd_merge_sort_keys(d.ptr, ctypes.byref(small), d.ptr, 1 << 20, i32, 0, dev.stream_ptr()) != 0
    assert lib.thrust_amd_merge_sort_keys(None, ctypes.byref(need), None, 10, 99, 0, dev.stream_ptr()) != 0
    assert lib.thrust_amd_merge_sort_pairs(None, ctypes.byref(need), None, None, 10, i32, 3, 0, dev.stream_ptr()) != 0


def test_merge_sort_full_size_properties(dev):
    """2^28 uint32 keys: sortedness, a 64-bit sum checksum and a histogram of the top byte; then
    2^27 pairs with 256 distinct keys, where stability fixes the order of the values: inside a
    run of equal keys the values (input positions) must increase.  All checked on the device."""
    import torch
    n = 1 << 28
    g = torch.Generator(device="cuda")
    g.manual_seed(11)
    src = torch.randint(-(1 << 31), 1 << 31, (n,), dtype=torch.int32, device="cuda", generator=g)

    def u32(t):
        return t.to(torch.int64) & 0xFFFFFFFF

    s_sum = int(u32(src).sum().item())
    s_hist = torch.bincount((u32(src) >> 24).to(torch.int64), minlength=256)
    d = dev.DeviceArray(n, dev.U32, src.view(torch.uint8).clone())
    del src
    dev.merge_sort_keys(d)
    o = u32(d.storage.view(torch.int32))
    assert bool((o[1:] >= o[:-1]).all().item())
    assert int(o.sum().item()) == s_sum
    assert torch.equal(torch.bincount((o >> 24).to(torch.int64), minlength=256), s_hist)
    del o, d

    m = 1 << 27
    keys = torch.randint(0, 256, (m,), dtype=torch.int32, device="cuda", generator=g)
    vals = torch.arange(m, dtype=torch.int32, device="cuda")
    counts = torch.bincount(keys.to(torch.int64), minlength=256)
    dk = dev.DeviceArray(m, dev.I32, keys.view(torch.uint8).clone())
    dv = dev.DeviceArray(m, dev.U32, vals.view(torch.uint8).clone())
    dev.merge_sort_pairs(dk, dv, descending=True)
    ok = dk.storage.view(torch.int32)
    ov = dv.storage.view(torch.int32)
    assert bool((ok[1:] <= ok[:-1]).all().item())
    assert torch.equal(torch.bincount(ok.to(torch.int64), minlength=256), counts)
    assert bool((keys[ov.to(torch.int64)] == ok).all().item())          # every value still sits with its key
    same = ok[1:] == ok[:-1]
    assert bool((ov[1:][same] > ov[:-1][same]).all().item())            # equal keys keep their input order
