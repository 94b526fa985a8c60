"""GPU test of thrust_amd_inclusive_scan_static, the entry point that allocates nothing.

Its output must be identical, bit for bit, to thrust_amd_inclusive_scan's (which the other
tests pin against the oracle) -- on two calls in a row, the second with a smaller input, so
that descriptors the first call left in the library's fixed scratch array cannot leak into
the second.  Sizes beyond the scratch array must be refused before anything is launched.
"""
import numpy as np
import pytest

from thrust_amd import datagen

pytestmark = pytest.mark.gpu


def _ints(n, dtype, seed):
    raw = datagen.splitmix64(seed, n)
    return raw.astype(dtype) if np.dtype(dtype).itemsize == 8 else (raw >> np.uint64(17)).astype(dtype)


@pytest.mark.parametrize("dtype,op", [(np.int32, 0), (np.uint64, 0), (np.int16, 2), (np.float32, 1)])
def test_static_scan_matches_the_temp_storage_entry_point(dev, oracle, dtype, op):
    # large-tile shape, a ragged last tile, then smaller inputs down to one element
    sizes = [(1 << 24) + 12345, (1 << 23) + 1, 100003, 4097, 1]
    for i, n in enumerate(sizes):
        if np.dtype(dtype).kind == "f":
            x = (datagen.splitmix64(31 + i, n) >> np.uint64(40)).astype(dtype) / dtype(1 << 12)
        else:
            x = _ints(n, dtype, 31 + i)
        d = dev.DeviceArray.from_numpy(x)
        want = dev.inclusive_scan(d, op=op).numpy()
        got = dev.inclusive_scan_static(d, op=op).numpy()
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), (dtype, op, n)
        if n <= 100003 and np.dtype(dtype).kind != "f":
            assert np.array_equal(got, oracle.inclusive_scan(x, op)), (dtype, op, n)
        if op == 0 and np.dtype(dtype).kind != "f":
            # every size against the definition as well: the running sum modulo 2^bits
            assert np.array_equal(got, np.cumsum(x, dtype=dtype)), (dtype, n)


def test_static_scan_in_place_and_empty(dev):
    x = _ints((1 << 22) + 3, np.int32, 5)
    d = dev.DeviceArray.from_numpy(x)
    want = dev.inclusive_scan(d).numpy()
    dev.inclusive_scan_static(d, out=d)
    assert np.array_equal(d.numpy(), want)
    empty = dev.DeviceArray.from_numpy(np.zeros(0, np.int32))
    dev.inclusive_scan_static(empty)  # n = 0: nothing to do, no error


def test_static_scan_refuses_sizes_beyond_its_scratch(dev):
    lib = dev.load()
    d = dev.DeviceArray.from_numpy(np.arange(16, dtype=np.int32))
    out = dev.DeviceArray(16, dev.I32)
    # 2^40 elements need more tile descriptors than the fixed array holds; the pointers are
    # never dereferenced because the call is refused before any launch
    # the library's launch log shows that nothing was launched by the refused calls
    dev.profile_collect()
    dev.profile_enable(True)
    try:
        rc = lib.thrust_amd_inclusive_scan_static(d.ptr, out.ptr, 1 << 40, dev.I32, dev.PLUS, dev.stream_ptr())
        assert rc != 0
        rc = lib.thrust_amd_inclusive_scan_static(d.ptr, out.ptr, 16, 99, dev.PLUS, dev.stream_ptr())
        assert rc != 0  # invalid dtype
        assert dev.profile_collect() == {}
    finally:
        dev.profile_enable(False)
    assert np.array_equal(d.numpy(), np.arange(16, dtype=np.int32))
    # and the entry point still works afterwards
    assert np.array_equal(dev.inclusive_scan_static(d).numpy(), np.cumsum(np.arange(16, dtype=np.int32)))


def test_static_scan_is_one_launch_and_calls_from_two_streams_follow_each_other(dev):
    import torch
    x = _ints((1 << 24) + 77, np.int32, 9)
    d = dev.DeviceArray.from_numpy(x)
    want = np.cumsum(x, dtype=np.int32)
    dev.profile_collect()
    dev.profile_enable(True)
    try:
        got = dev.inclusive_scan_static(d).numpy()
        log = dev.profile_collect()
    finally:
        dev.profile_enable(False)
    assert np.array_equal(got, want)
    assert sum(v[0] for v in log.values()) == 1, log  # the scan kernel alone: no clearing launch
    # calls issued on two streams without any synchronisation in between share the scratch array;
    # the library puts them one behind the other
    lib = dev.load()
    outs = [dev.DeviceArray(d.n, dev.I32) for _ in range(6)]
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    torch.cuda.synchronize()
    for i, o in enumerate(outs):
        rc = lib.thrust_amd_inclusive_scan_static(d.ptr, o.ptr, d.n, dev.I32, dev.PLUS, streams[i % 2].cuda_stream)
        assert rc == 0
    torch.cuda.synchronize()
    for o in outs:
        assert np.array_equal(o.numpy(), want)
