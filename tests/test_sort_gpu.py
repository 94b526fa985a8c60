"""GPU parity: thrust_amd_sort_keys / thrust_amd_sort_pairs against the CPU oracle.

Sort results have a unique answer (total order on the radix encoding; stability fixes
the order of values of equal keys), so everything is compared bit for bit -- floats
through their bit patterns, against the one-thread oracle (= the reference's CPP
system; the multi-thread OMP layout of +-0.0 depends on the thread count).
Mirrors testing/sort.cu:80-90, testing/stable_sort_by_key.cu:99-116 and
testing/sort_variable_bits.cu:18-43.
"""
import numpy as np
import pytest

from thrust_amd import datagen

pytestmark = pytest.mark.gpu

SIZES = [0, 1, 2, 63, 64, 65, 1000, 4096, 8191, 8192, 8193, 16383, 16384, 16385, 65537, 100003,
         (1 << 20) + 13]
KEY_DTYPES = [np.int8, np.uint8, np.int16, np.uint16, np.int32, np.uint32, np.int64, np.uint64,
              np.float32, np.float64]


def _keys(n, dtype, seed):
    raw = datagen.splitmix64(seed, n)
    dt = np.dtype(dtype)
    if dt.kind == "f":
        u = raw if dt.itemsize == 8 else (raw >> np.uint64(32)).astype(np.uint32)
        f = u.view(dtype).copy()
        f[~np.isfinite(f)] = 0  # NaN/inf patterns are exercised separately
        return f
    return raw.astype(dtype) if dt.itemsize == 8 else (raw >> np.uint64(13)).astype(dtype)


def _bits(a):
    return a.view({1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}[a.dtype.itemsize])


@pytest.mark.parametrize("dtype", KEY_DTYPES)
def test_sort_keys_all_types(dev, oracle_seq, dtype):
    for n in SIZES:
        k = _keys(n, dtype, 3)
        d = dev.DeviceArray.from_numpy(k)
        dev.sort_keys(d)
        assert np.array_equal(_bits(d.numpy()), _bits(oracle_seq.sort_keys(k))), (dtype, n)


@pytest.mark.parametrize("dtype", [np.int32, np.uint32, np.float32, np.uint64, np.float64])
def test_sort_keys_descending(dev, oracle_seq, dtype):
    for n in [1, 77, 16385, 100003]:
        k = _keys(n, dtype, 5)
        d = dev.DeviceArray.from_numpy(k)
        dev.sort_keys(d, descending=True)
        assert np.array_equal(_bits(d.numpy()), _bits(oracle_seq.sort_keys(k, descending=True)))


def test_sort_float_special_values(dev, oracle_seq):
    n = 70001
    k = datagen.c2_float32(n)
    k[::997] = np.float32("nan")
    k[5::997] = -np.float32("nan")
    k[7::997] = np.float32("inf")
    k[9::997] = -np.float32("inf")
    d = dev.DeviceArray.from_numpy(k)
    dev.sort_keys(d)
    assert np.array_equal(_bits(d.numpy()), _bits(oracle_seq.sort_keys(k)))


@pytest.mark.parametrize("kdtype", [np.uint32, np.int32, np.float32, np.uint64, np.int64, np.uint16])
@pytest.mark.parametrize("vdtype", [np.uint32, np.uint64])
def test_sort_pairs_stable(dev, oracle_seq, kdtype, vdtype):
    for n in [0, 1, 1000, 8193, 16385, 100003, (1 << 19) + 5]:
        k = _keys(n, kdtype, 7)
        if n > 10:
            k[1::3] = k[0]  # many duplicates: stability becomes visible in the values
        v = np.arange(n, dtype=vdtype)
        dk, dv = dev.DeviceArray.from_numpy(k), dev.DeviceArray.from_numpy(v)
        dev.sort_pairs(dk, dv)
        rk, rv = oracle_seq.sort_pairs(k, v)
        assert np.array_equal(_bits(dk.numpy()), _bits(rk)), (kdtype, n)
        assert np.array_equal(dv.numpy(), rv), (kdtype, n)


def test_sort_pairs_descending_is_stable(dev, oracle_seq):
    n = 50001
    k = (_keys(n, np.uint32, 9) % 50).astype(np.uint32)
    v = np.arange(n, dtype=np.uint32)
    dk, dv = dev.DeviceArray.from_numpy(k), dev.DeviceArray.from_numpy(v)
    dev.sort_pairs(dk, dv, descending=True)
    rk, rv = oracle_seq.sort_pairs(k, v, descending=True)
    assert np.array_equal(dk.numpy(), rk) and np.array_equal(dv.numpy(), rv)


def test_sort_variable_bits(dev):
    """Keys masked to their low b bits (testing/sort_variable_bits.cu:18-43): skipped passes."""
    n = 40001
    for b in [0, 1, 7, 8, 9, 16, 21, 32]:
        k = _keys(n, np.uint32, 11) & np.uint32((1 << b) - 1 if b < 32 else 0xFFFFFFFF)
        d = dev.DeviceArray.from_numpy(k)
        dev.sort_keys(d)
        assert np.array_equal(d.numpy(), np.sort(k, kind="stable")), b


def test_sort_bit_range(dev):
    n = 30001
    k = _keys(n, np.uint32, 13)
    v = np.arange(n, dtype=np.uint32)
    for lo, hi in [(0, 8), (4, 20), (8, 32), (5, 6), (12, 12)]:
        dk, dv = dev.DeviceArray.from_numpy(k), dev.DeviceArray.from_numpy(v)
        dev.sort_pairs(dk, dv, begin_bit=lo, end_bit=hi)
        digit = (k.astype(np.uint64) >> np.uint64(lo)) & np.uint64((1 << (hi - lo)) - 1)
        order = np.argsort(digit, kind="stable")
        assert np.array_equal(dk.numpy(), k[order]) and np.array_equal(dv.numpy(), v[order])


@pytest.mark.parametrize("kind", ["full", "low16", "skew90"])
def test_config3_key_distributions(dev, oracle_seq, kind):
    n = (1 << 21) + 17
    k = datagen.c3_uint64(n, kind)
    v = np.arange(n, dtype=np.uint32)
    dk, dv = dev.DeviceArray.from_numpy(k), dev.DeviceArray.from_numpy(v)
    dev.sort_pairs(dk, dv)
    rk, rv = oracle_seq.sort_pairs(k, v)
    assert np.array_equal(dk.numpy(), rk) and np.array_equal(dv.numpy(), rv)


@pytest.mark.parametrize("kind", ["full", "low16", "skew90"])
def test_config3_full_size_properties(dev, kind):
    """Config 3 at its own size, N = 2^27 uint64 keys with uint32 values = original index
    (testing/stable_sort_by_key.cu:99-116 at the configuration's size).  Checked on the device:
    keys ascending, the values a permutation of 0..n-1, every value still carrying its key
    (keys_in[values_out] == keys_out) and values ascending inside every run of equal keys.
    Together these fix the output completely: it is the stable sort of the input."""
    import torch
    n = 1 << 27
    k = datagen.c3_uint64(n, kind)
    keys_in = torch.from_numpy(k.view(np.int64)).cuda()
    del k
    dk = dev.DeviceArray(n, dev.U64, keys_in.view(torch.uint8).clone())
    dv = dev.DeviceArray(n, dev.U32, torch.arange(n, dtype=torch.int32, device="cuda").view(torch.uint8))
    dev.sort_pairs(dk, dv)
    ko = dk.storage.view(torch.int64)
    vo = dv.storage.view(torch.int32).to(torch.int64)  # indices below 2^27: non-negative
    flip = torch.tensor(-(1 << 63), dtype=torch.int64, device="cuda")
    ordered = ko ^ flip  # unsigned order as signed order
    assert bool((ordered[1:] >= ordered[:-1]).all().item()), kind
    seen = torch.zeros(n, dtype=torch.bool, device="cuda")
    seen[vo] = True
    assert bool(seen.all().item()), kind
    assert bool((keys_in[vo] == ko).all().item()), kind
    same = ko[1:] == ko[:-1]
    assert bool((vo[1:][same] > vo[:-1][same]).all().item()), kind
    if kind == "low16":
        assert int(ko.max().item()) <= 0xFFFF
    if kind == "skew90":
        frac = float((ko == datagen.C3_CONSTANT).sum().item()) / n
        assert 0.89 < frac < 0.91


def test_config2_full_size_properties(dev):
    """Config 2 at N=2^28: sortedness, multiset preservation (histogram of all bytes and a
    64-bit sum/xor checksum) for uint32; the float32 case is checked on its encoded bits."""
    n = 1 << 28
    for gen in (datagen.c2_uint32, datagen.c2_float32):
        k = gen(n)
        d = dev.DeviceArray.from_numpy(k)
        dev.sort_keys(d)
        out = d.numpy()
        b_in, b_out = _bits(k), _bits(out)
        if k.dtype == np.float32:
            enc = lambda u: u ^ (np.where(u >> 31, np.uint32(0xFFFFFFFF), np.uint32(0x80000000)))
            e_out = enc(b_out)
        else:
            e_out = b_out
        assert np.all(e_out[:-1] <= e_out[1:])
        assert int(np.sum(b_in, dtype=np.uint64)) == int(np.sum(b_out, dtype=np.uint64))
        assert int(np.bitwise_xor.reduce(b_in)) == int(np.bitwise_xor.reduce(b_out))
        assert np.array_equal(np.bincount(b_in >> 20, minlength=4096),
                              np.bincount(b_out >> 20, minlength=4096))


def test_sort_beyond_2p30_keys_properties(dev):
    """More than 2^30 keys take the 64-bit tile descriptors: sortedness, a 64-bit sum / xor
    checksum and a byte histogram of the keys, and stability through the values, all checked
    on the device (keys generated there from a seeded generator)."""
    import torch
    n = (1 << 30) + 12345
    g = torch.Generator(device="cuda")
    g.manual_seed(7)
    src = torch.randint(-(1 << 31), 1 << 31, (n,), dtype=torch.int32, device="cuda", generator=g)

    def u32(t):  # int32 bits as non-negative int64
        return t.to(torch.int64) & 0xFFFFFFFF

    s_sum = int(u32(src).sum().item())
    s_hist = torch.bincount((u32(src) >> 24).to(torch.int64), minlength=256)
    d = dev.DeviceArray(n, dev.U32, src.view(torch.uint8).clone())
    dev.sort_keys(d)
    out = d.storage.view(torch.int32)
    o = u32(out)
    assert bool((o[1:] >= o[:-1]).all().item())
    assert int(o.sum().item()) == s_sum
    assert torch.equal(torch.bincount((o >> 24).to(torch.int64), minlength=256), s_hist)
    del o, d, out
    # pairs with only 8 significant key bits: one pass, and the values of equal keys must
    # stay in their input order
    keys = (src & 0xFF).to(torch.int32)
    vals = torch.arange(n, dtype=torch.int32, device="cuda")
    dk = dev.DeviceArray(n, dev.U32, keys.view(torch.uint8).clone())
    dv = dev.DeviceArray(n, dev.U32, vals.view(torch.uint8))
    dev.sort_pairs(dk, dv)
    ko = dk.storage.view(torch.int32)
    vo = dv.storage.view(torch.int32)
    assert bool((ko[1:] >= ko[:-1]).all().item())
    same = ko[1:] == ko[:-1]
    assert bool((vo[1:][same] > vo[:-1][same]).all().item())  # ascending inside every key: stable
    assert bool((keys[vo.to(torch.int64)] == ko).all().item())  # every value still carries its key


def test_sorts_in_flight_on_several_streams(dev):
    """Twelve sorts issued on four streams without any synchronisation in between share the device:
    the passes of different calls run side by side, each with a part of the workgroup slots, and each
    call's tiles still find their predecessors (the ticket rule of the passes must not depend on a
    call having the device to itself)."""
    import torch
    sizes = [(1 << 22) + 5, (1 << 21) + 12345, 3000017]
    streams = [torch.cuda.Stream() for _ in range(4)]
    jobs = []
    for si, st in enumerate(streams):
        for ni, n in enumerate(sizes):
            k = _keys(n, np.uint32, 100 + 10 * si + ni)
            v = np.arange(n, dtype=np.uint32)
            jobs.append((st, k, dev.DeviceArray.from_numpy(k), dev.DeviceArray.from_numpy(v), dev.Temp()))
    for st, k, dk, dv, t in jobs:  # sizes the temporary storage of every job: no allocation in the timed part
        with torch.cuda.stream(st):
            dev.sort_pairs(dev.DeviceArray.from_numpy(k), dev.DeviceArray.from_numpy(np.arange(k.size, dtype=np.uint32)), temp=t)
    torch.cuda.synchronize()
    for st, k, dk, dv, t in jobs:
        with torch.cuda.stream(st):
            dev.sort_pairs(dk, dv, temp=t)
    torch.cuda.synchronize()
    for st, k, dk, dv, t in jobs:
        order = np.argsort(k, kind="stable")
        assert np.array_equal(dk.numpy(), k[order])
        assert np.array_equal(dv.numpy(), order.astype(np.uint32))

