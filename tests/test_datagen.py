"""The device-side input generators (torch, int64 arithmetic) must produce the same bytes as
the numpy generators the CPU baseline and the fixtures use.  Runs torch on the CPU."""
import numpy as np
import torch

from thrust_amd import datagen as d
from thrust_amd import datagen_device as dd

N = 100003


def test_streams_match_numpy_generators():
    assert np.array_equal(dd.splitmix64(torch, 7, N, 5, "cpu").numpy().view(np.uint64), d.splitmix64(7, N, 5))
    assert np.array_equal(dd.c1_int32(torch, N, device="cpu").numpy(), d.c1_int32(N))
    assert np.array_equal(dd.c2_uint32(torch, N, device="cpu").numpy().view(np.uint32), d.c2_uint32(N))
    assert np.array_equal(dd.c2_float32(torch, N, device="cpu").numpy().view(np.uint32),
                          d.c2_float32(N).view(np.uint32))
    for kind in ("full", "low16", "skew90"):
        assert np.array_equal(dd.c3_uint64(torch, N, kind, device="cpu").numpy().view(np.uint64),
                              d.c3_uint64(N, kind))
    assert np.array_equal(dd.c5_float32(torch, N, device="cpu").numpy(), d.c5_float32(N))


def test_merge_inputs_match_and_segments_are_well_formed():
    (a, va), (b, vb) = dd.c5_merge_inputs(torch, 5000, device="cpu")
    (ra, rva), (rb, rvb) = d.c5_merge_inputs(5000)
    assert np.array_equal(a.numpy().view(np.uint32), ra) and np.array_equal(va.numpy().view(np.uint32), rva)
    assert np.array_equal(b.numpy().view(np.uint32), rb) and np.array_equal(vb.numpy().view(np.uint32), rvb)
    keys, vals = dd.c4_segments(torch, N, 8, device="cpu")
    k = keys.numpy()
    assert k[0] == 0 and np.all(np.diff(k) >= 0) and np.all(np.diff(k) <= 1)
    assert 6.0 < N / (k[-1] + 1) < 10.0  # mean run length about 8
    assert np.array_equal(vals.numpy(), d.c4_segments(N, 8)[1])
