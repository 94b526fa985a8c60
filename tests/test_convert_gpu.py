"""GPU parity: thrust_amd_convert, and the reference's mixed-element-type rules for reduce
and the scans composed from it through the C ABI, against the CPU oracle.

The reference accumulates reduce and exclusive_scan in the type of init and inclusive_scan
in the type of the input, converting elements on the way in and results on the way out
(testing/reduce.cu:98-129, testing/scan.cu:236-297).  Conversions are C's: truncation
toward zero from floating point, wrap-around into narrower integers; every value here is
in the range of its target where C leaves the result open.
"""
import json
import os

import numpy as np
import pytest

from thrust_amd import datagen

pytestmark = pytest.mark.gpu

SIZES = [0, 1, 2, 63, 64, 65, 1000, 4095, 4096, 4097, 100003, (1 << 20) + 13, (1 << 22) + 5]
DTYPES = [np.int8, np.uint8, np.int16, np.uint16, np.int32, np.uint32, np.int64, np.uint64, np.float32, np.float64]
KA = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "known_answers.json")))


def _source(n, dtype, seed, unsigned_target):
    raw = datagen.splitmix64(seed, n)
    if np.dtype(dtype).kind == "f":
        # multiples of 1/8: float64 sums of these are exact in every association order
        x = (raw % np.uint64(1601)).astype(np.float64) / 8.0 - (0.0 if unsigned_target else 100.0)
        return x.astype(dtype)
    return raw.astype(dtype)  # integers: all bit patterns, conversions between integers wrap


def _reduce_as(dev, d, init, op):
    init = np.asarray(init)
    return dev.reduce(dev.convert(d, dev.DTYPE_OF_NP[init.dtype]), op=op, init=init[()]).numpy()[0]


def _inclusive_scan_as(dev, d, out_dtype, op):
    return dev.convert(dev.inclusive_scan(d, op=op), dev.DTYPE_OF_NP[np.dtype(out_dtype)]).numpy()


def _exclusive_scan_as(dev, d, init, out_dtype, op):
    init = np.asarray(init)
    acc = dev.convert(d, dev.DTYPE_OF_NP[init.dtype])
    return dev.convert(dev.exclusive_scan(acc, init=init[()], op=op), dev.DTYPE_OF_NP[np.dtype(out_dtype)]).numpy()


@pytest.mark.parametrize("src", DTYPES)
def test_convert_every_pair(dev, oracle, src):
    for dst in DTYPES:
        int_target = np.dtype(dst).kind != "f"
        for n in (0, 1, 63, 4097, 100003):
            x = _source(n, src, 61, int_target and np.dtype(dst).kind == "u")
            if np.dtype(src).kind == "f" and int_target and np.dtype(dst).itemsize == 1:
                x = np.clip(x, 0 if np.dtype(dst).kind == "u" else -100, 100).astype(src)
            got = dev.convert(dev.DeviceArray.from_numpy(x), dev.DTYPE_OF_NP[np.dtype(dst)]).numpy()
            want = oracle.convert(x, dst)
            assert got.dtype == want.dtype and got.tobytes() == want.tobytes(), (src, dst, n)


def test_convert_large_and_in_place_widths(dev, oracle):
    for n in SIZES:
        x = _source(n, np.int32, 62, False)
        d = dev.DeviceArray.from_numpy(x)
        assert np.array_equal(dev.convert(d, dev.DTYPE_OF_NP[np.dtype(np.int64)]).numpy(), x.astype(np.int64)), n
        assert np.array_equal(dev.convert(d, dev.DTYPE_OF_NP[np.dtype(np.uint8)]).numpy(), x.astype(np.uint8)), n
        # same width, same buffer: every element is read before it is written by the same lane
        same = dev.convert(d, dev.DTYPE_OF_NP[np.dtype(np.float32)], out=dev.DeviceArray(n, dev.DTYPE_OF_NP[np.dtype(np.float32)], d.storage))
        assert same.numpy().tobytes() == oracle.convert(x, np.float32).tobytes(), n


def test_mixed_known_answers(dev):
    for c in KA["reduce_mixed"]:
        init = np.dtype(c["init_dtype"]).type(c["init"])
        d = dev.DeviceArray.from_numpy(np.array(c["in"], c["in_dtype"]))
        got = _reduce_as(dev, d, init, dev.PLUS)
        assert got.dtype == init.dtype and got == c["out"], c["source"]
    for c in KA["scan_mixed"]:
        d = dev.DeviceArray.from_numpy(np.array(c["in"], c["in_dtype"]))
        if c["kind"] == "inclusive":
            got = _inclusive_scan_as(dev, d, c["out_dtype"], dev.PLUS)
        else:
            got = _exclusive_scan_as(dev, d, np.dtype(c["init_dtype"]).type(c["init"]), c["out_dtype"], dev.PLUS)
        assert got.dtype == np.dtype(c["out_dtype"]) and got.tolist() == c["out"], c["source"]


@pytest.mark.parametrize("pair", [(np.float32, np.int32), (np.int16, np.int64), (np.uint8, np.uint32),
                                  (np.int32, np.float64), (np.float64, np.int64), (np.int64, np.int8)])
def test_mixed_reduce_and_scans_match_oracle(dev, oracle, pair):
    src, acc = pair
    exact = np.dtype(acc).kind != "f"
    for n in SIZES:
        x = _source(n, src, 63, np.dtype(acc).kind == "u")
        if np.dtype(src).kind != "f":
            x = (x.astype(np.int64) % 2001 - (0 if np.dtype(src).kind == "u" else 1000)).astype(src)
        d = dev.DeviceArray.from_numpy(x)
        init = np.dtype(acc).type(5)
        for op in (dev.PLUS, dev.MAX):
            got, want = _reduce_as(dev, d, init, op), oracle.reduce_as(x, init, op)
            assert got == want if exact else abs(float(got) - float(want)) <= 1e-9 * max(1.0, abs(float(want))), (pair, n, op)
            got, want = _exclusive_scan_as(dev, d, init, src, op), oracle.exclusive_scan_as(x, init, src, op)
            if exact or np.dtype(src).kind != "f":
                # integer accumulators are exact; a float64 accumulator over integers below 2^53 is too
                assert got.tobytes() == want.tobytes(), ("exclusive", pair, n, op)
            got, want = _inclusive_scan_as(dev, d, acc, op), oracle.inclusive_scan_as(x, acc, op)
            if np.dtype(src) != np.dtype(np.float32) or op == dev.MAX:
                assert got.tobytes() == want.tobytes(), ("inclusive", pair, n, op)
            elif n:
                # float32 accumulator, integer output: the association order shows in the last
                # bits of the sums and truncation carries that into the integers
                err = np.max(np.abs(got.astype(np.float64) - want.astype(np.float64)))
                assert err <= 1.0 + 2e-4 * np.max(np.abs(want.astype(np.float64))), (pair, n, op)


def test_convert_rejects_bad_arguments(dev):
    lib = dev.load()
    d = dev.DeviceArray(16, dev.DTYPE_OF_NP[np.dtype(np.int32)])
    assert lib.thrust_amd_convert(d.ptr, 99, d.ptr, 0, 16, dev.stream_ptr()) != 0
    assert lib.thrust_amd_convert(d.ptr, 0, d.ptr, -1, 16, dev.stream_ptr()) != 0
    assert lib.thrust_amd_convert(None, 0, d.ptr, 0, 16, dev.stream_ptr()) != 0
    assert lib.thrust_amd_convert(None, 0, None, 0, 0, dev.stream_ptr()) == 0


@pytest.mark.parametrize("dtype", DTYPES)
def test_sequence_every_type(dev, dtype):
    # thrust::sequence(first, last, init, step): element i is (T)(init + step * (T)i)
    # (thrust/system/detail/generic/sequence.inl:56-85; testing/sequence.cu:43-76 for the literal cases)
    t = np.dtype(dtype)
    cases = [(0, 1), (10, 2), (3, 7)] if t.kind != "f" else [(0.0, 1.0), (10.0, 2.0), (0.1, 0.3), (-1.5, 1e-3)]
    if t.kind == "i":
        cases.append((-5, -3))
    for n in (0, 1, 5, 63, 4097, 100003):
        i = np.arange(n, dtype=np.uint64).astype(t)  # (T)i: wraps for the narrow types
        for init, step in cases:
            with np.errstate(over="ignore"):
                if t.kind == "f":
                    want = t.type(init) + t.type(step) * i  # every operation rounded to T, no fused multiply-add
                else:
                    wide = np.int64 if t.kind == "i" else np.uint64
                    want = (wide(init) + wide(step) * i.astype(wide)).astype(t)
            got = dev.sequence(n, dev.DTYPE_OF_NP[t], init, step).numpy()
            assert got.dtype == want.dtype and got.tobytes() == want.tobytes(), (dtype, n, init, step)
    got = dev.sequence(5, dev.DTYPE_OF_NP[t], 10, 2).numpy()
    assert list(got) == [10, 12, 14, 16, 18]
    lib = dev.load()
    assert lib.thrust_amd_sequence(None, 0, dev.DTYPE_OF_NP[t], None, None, dev.stream_ptr()) == 0
    assert lib.thrust_amd_sequence(None, 4, dev.DTYPE_OF_NP[t], None, None, dev.stream_ptr()) != 0
    assert lib.thrust_amd_sequence(got.ctypes.data, 4, 99, got.ctypes.data, got.ctypes.data, dev.stream_ptr()) != 0
