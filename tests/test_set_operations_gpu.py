"""GPU parity: thrust_amd_set_operation and thrust_amd_set_operation_by_key against the CPU
oracle (bit-exact: keys, the side every kept element comes from, and the values).

Models: testing/set_{difference,intersection,symmetric_difference,union}.cu (simple vectors,
equivalent elements, random inputs of all sizes), their *_descending.cu and *_by_key.cu forms.
"""
import numpy as np
import pytest

from thrust_amd import datagen

pytestmark = pytest.mark.gpu

OPS = [0, 1, 2, 3]  # difference, intersection, symmetric difference, union
SIZES = [(0, 0), (0, 5), (5, 0), (1, 1), (3, 4), (100, 1), (4095, 1), (4096, 4096), (4097, 4095), (8191, 1),
         (10000, 777), (50000, 50001), (1 << 18, (1 << 17) + 5)]


def _sorted(n, dtype, seed, spread, descending=False):
    """n sorted values with runs of duplicates: about n / spread distinct keys."""
    raw = datagen.splitmix64(seed, n) % np.uint64(max(n // spread, 1) + 1)
    x = np.sort(raw.astype(dtype))  # narrow types wrap first, then sort
    return x[::-1].copy() if descending else x


@pytest.mark.parametrize("dtype", [np.int32, np.uint8, np.uint64, np.float32, np.int16, np.float64])
@pytest.mark.parametrize("op", OPS)
def test_set_operation_sizes(dev, oracle, dtype, op):
    for na, nb in SIZES:
        spread = 1 if np.dtype(dtype).itemsize == 1 else 3
        a, b = _sorted(na, dtype, 71, spread), _sorted(nb, dtype, 72, spread)
        out, cnt = dev.set_operation(op, dev.DeviceArray.from_numpy(a), dev.DeviceArray.from_numpy(b))
        ref = oracle.set_operation(op, a, b)
        assert cnt == ref.size and np.array_equal(out.numpy()[:cnt], ref), (dtype, op, na, nb)


@pytest.mark.parametrize("op", OPS)
def test_set_operation_known_answers(dev, op):
    # testing/set_difference.cu:70-80, set_intersection.cu:71-81, set_symmetric_difference.cu:70-80,
    # set_union.cu:71-81 and :96-106 (equivalent elements)
    cases = {
        0: [([0, 2, 4, 5], [0, 3, 3, 4, 6], [2, 5])],
        1: [([0, 2, 4], [0, 3, 3, 4], [0, 4])],
        2: [([0, 2, 4, 6], [0, 3, 3, 4, 7], [2, 3, 3, 6, 7])],
        3: [([0, 2, 4], [0, 3, 3, 4], [0, 2, 3, 3, 4]), ([0, 2, 2], [0, 2, 2, 2, 3], [0, 2, 2, 2, 3])],
    }
    for a, b, ref in cases[op]:
        out, cnt = dev.set_operation(op, dev.DeviceArray.from_numpy(np.array(a, np.int32)),
                                     dev.DeviceArray.from_numpy(np.array(b, np.int32)))
        assert out.numpy()[:cnt].tolist() == ref


@pytest.mark.parametrize("op", OPS)
def test_set_operation_descending(dev, oracle, op):
    # testing/set_union_descending.cu:7-18
    if op == 3:
        out, cnt = dev.set_operation(op, dev.DeviceArray.from_numpy(np.array([4, 2, 0], np.int32)),
                                     dev.DeviceArray.from_numpy(np.array([4, 3, 3, 0], np.int32)), descending=True)
        assert out.numpy()[:cnt].tolist() == [4, 3, 3, 2, 0]
    for na, nb in [(7, 9), (5000, 4097), (70001, 30000)]:
        a, b = _sorted(na, np.int32, 73, 4, True), _sorted(nb, np.int32, 74, 4, True)
        out, cnt = dev.set_operation(op, dev.DeviceArray.from_numpy(a), dev.DeviceArray.from_numpy(b), descending=True)
        ref = oracle.set_operation(op, a, b, True)
        assert cnt == ref.size and np.array_equal(out.numpy()[:cnt], ref), (op, na, nb)


@pytest.mark.parametrize("op", OPS)
def test_set_operation_long_runs_across_tiles(dev, oracle, op):
    """Runs of equal keys much longer than a tile (8192 merged elements for 4-byte keys), in
    one range, in both, and ending exactly on tile borders."""
    shapes = [
        (np.zeros(20000, np.int32), np.zeros(9000, np.int32)),
        (np.zeros(9000, np.int32), np.zeros(20000, np.int32)),
        (np.repeat(np.arange(4, dtype=np.int32), 4096), np.repeat(np.arange(4, dtype=np.int32), 4096)),
        (np.repeat(np.arange(3, dtype=np.int32), [5000, 1, 7000]), np.repeat(np.arange(1, 4, dtype=np.int32), [3000, 6000, 2])),
        (np.r_[np.zeros(4096, np.int32), np.ones(100, np.int32)], np.r_[np.ones(4096, np.int32), np.full(3, 2, np.int32)]),
        (np.repeat(np.arange(4, dtype=np.int32), 8192), np.repeat(np.arange(4, dtype=np.int32), 8192)),
        (np.r_[np.zeros(8192, np.int32), np.ones(100, np.int32)], np.r_[np.ones(8192, np.int32), np.full(3, 2, np.int32)]),
        (np.repeat(np.arange(3, dtype=np.int32), [30000, 1, 17000]), np.repeat(np.arange(1, 4, dtype=np.int32), [9000, 26000, 2])),
        (np.arange(12288, dtype=np.int32), np.arange(12288, dtype=np.int32)),
        (np.arange(0, 24576, 2, dtype=np.int32), np.arange(1, 24576, 2, dtype=np.int32)),
    ]
    for a, b in shapes:
        out, cnt = dev.set_operation(op, dev.DeviceArray.from_numpy(a), dev.DeviceArray.from_numpy(b))
        ref = oracle.set_operation(op, a, b)
        assert cnt == ref.size and np.array_equal(out.numpy()[:cnt], ref), (op, a.size, b.size)


@pytest.mark.parametrize("vdtype", [np.uint32, np.uint64, np.uint8, np.uint16])
@pytest.mark.parametrize("op", OPS)
def test_set_operation_by_key(dev, oracle, op, vdtype):
    # known answers: testing/set_union_by_key.cu:89-104, set_symmetric_difference_by_key.cu:89-104
    if op == 3 and vdtype == np.uint32:
        ka, kb = np.array([0, 2, 4], np.int32), np.array([0, 3, 3, 4], np.int32)
        ko, vo, cnt = dev.set_operation_by_key(op, dev.DeviceArray.from_numpy(ka), dev.DeviceArray.from_numpy(kb),
                                               dev.DeviceArray.from_numpy(np.zeros(3, vdtype)),
                                               dev.DeviceArray.from_numpy(np.ones(4, vdtype)))
        assert ko.numpy()[:cnt].tolist() == [0, 2, 3, 3, 4] and vo.numpy()[:cnt].tolist() == [0, 0, 1, 1, 0]
    for na, nb in [(0, 3), (3, 0), (5, 7), (4096, 4096), (30000, 12345), (1 << 17, 1 << 17)]:
        ka, kb = _sorted(na, np.int32, 75, 3), _sorted(nb, np.int32, 76, 3)
        # values name their origin: index, plus a high bit for the second range
        top = np.uint64(1) << np.uint64(8 * np.dtype(vdtype).itemsize - 1)
        va = (np.arange(na, dtype=np.uint64) % top).astype(vdtype)
        vb = ((np.arange(nb, dtype=np.uint64) % top) + top).astype(vdtype)
        ko, vo, cnt = dev.set_operation_by_key(op, dev.DeviceArray.from_numpy(ka), dev.DeviceArray.from_numpy(kb),
                                               dev.DeviceArray.from_numpy(va), dev.DeviceArray.from_numpy(vb))
        rk, rv = oracle.set_operation_by_key(op, ka, kb, va, vb)
        assert cnt == rk.size and np.array_equal(ko.numpy()[:cnt], rk) and np.array_equal(vo.numpy()[:cnt], rv), (op, na, nb)


def _origin_values(na, nb, vdtype=np.uint32):
    """Values that name their origin: the index, plus the top bit for the second range."""
    top = np.uint64(1) << np.uint64(8 * np.dtype(vdtype).itemsize - 1)
    va = (np.arange(na, dtype=np.uint64) % top).astype(vdtype)
    vb = ((np.arange(nb, dtype=np.uint64) % top) + top).astype(vdtype)
    return va, vb


@pytest.mark.parametrize("op", OPS)
def test_set_operation_by_key_long_runs_name_the_surviving_copies(dev, oracle, op):
    """Runs longer than a tile, starting before a tile and ending after it, in A, in B and in both:
    the values tell which copies of the equal keys were kept."""
    shapes = [
        (np.zeros(20000, np.int32), np.zeros(9000, np.int32)),
        (np.zeros(9000, np.int32), np.zeros(20000, np.int32)),
        (np.repeat(np.arange(3, dtype=np.int32), [5000, 1, 7000]), np.repeat(np.arange(1, 4, dtype=np.int32), [3000, 6000, 2])),
        (np.r_[np.zeros(8192, np.int32), np.ones(100, np.int32)], np.r_[np.ones(8192, np.int32), np.full(3, 2, np.int32)]),
        (np.repeat(np.arange(3, dtype=np.int32), [30000, 1, 17000]), np.repeat(np.arange(1, 4, dtype=np.int32), [9000, 26000, 2])),
        (np.repeat(np.arange(6, dtype=np.int32), [8190, 3, 8192, 1, 16384, 5]), np.repeat(np.arange(6, dtype=np.int32), [2, 8191, 1, 8192, 7, 16390])),
        (np.repeat(np.arange(700, dtype=np.int32), 13), np.repeat(np.arange(700, dtype=np.int32), 17)),
    ]
    for ka, kb in shapes:
        va, vb = _origin_values(ka.size, kb.size)
        ko, vo, cnt = dev.set_operation_by_key(op, dev.DeviceArray.from_numpy(ka), dev.DeviceArray.from_numpy(kb),
                                               dev.DeviceArray.from_numpy(va), dev.DeviceArray.from_numpy(vb))
        rk, rv = oracle.set_operation_by_key(op, ka, kb, va, vb)
        assert cnt == rk.size and np.array_equal(ko.numpy()[:cnt], rk) and np.array_equal(vo.numpy()[:cnt], rv), (op, ka.size, kb.size)


@pytest.mark.parametrize("kdtype", [np.uint64, np.float64, np.int16, np.uint8])
@pytest.mark.parametrize("op", OPS)
def test_set_operation_by_key_other_key_widths_and_descending(dev, oracle, op, kdtype):
    """8-byte keys take the 256-thread tile, 1- and 2-byte keys repeat themselves by the thousand."""
    for na, nb, descending in [(5, 7, False), (4096, 4097, False), (40000, 23456, True), (1 << 16, (1 << 16) + 3, False)]:
        spread = 1 if np.dtype(kdtype).itemsize == 1 else 3
        ka, kb = _sorted(na, kdtype, 77, spread, descending), _sorted(nb, kdtype, 78, spread, descending)
        va, vb = _origin_values(na, nb)
        ko, vo, cnt = dev.set_operation_by_key(op, dev.DeviceArray.from_numpy(ka), dev.DeviceArray.from_numpy(kb),
                                               dev.DeviceArray.from_numpy(va), dev.DeviceArray.from_numpy(vb),
                                               descending=descending)
        rk, rv = oracle.set_operation_by_key(op, ka, kb, va, vb, descending)
        assert cnt == rk.size and np.array_equal(ko.numpy()[:cnt], rk) and np.array_equal(vo.numpy()[:cnt], rv), (op, kdtype, na, nb)


@pytest.mark.parametrize("op", OPS)
def test_set_operation_mostly_distinct_keys_with_a_few_repeated(dev, oracle, op):
    """Ranges that are sets but for a few hundred keys with multiplicities 0..3 on either side:
    nearly every wave decides its elements without counting, the planted keys land anywhere
    (inside lanes, across lanes, waves and tiles) and must be counted."""
    for seed in (91, 92, 93):
        pool = np.unique(datagen.splitmix64(seed, 300000) >> np.uint64(33)).astype(np.uint32)
        side = datagen.splitmix64(seed + 10, pool.size) % np.uint64(4)  # 0: A only, 1: B only, 2 and 3: both
        ma = (side != 1).astype(np.int64)
        mb = (side != 0).astype(np.int64)
        planted = (datagen.splitmix64(seed + 20, 400) % np.uint64(pool.size)).astype(np.int64)
        ma[planted] = (datagen.splitmix64(seed + 30, 400) % np.uint64(4)).astype(np.int64)
        mb[planted] = (datagen.splitmix64(seed + 40, 400) % np.uint64(4)).astype(np.int64)
        a, b = np.repeat(pool, ma), np.repeat(pool, mb)
        va, vb = _origin_values(a.size, b.size)
        ko, vo, cnt = dev.set_operation_by_key(op, dev.DeviceArray.from_numpy(a), dev.DeviceArray.from_numpy(b),
                                               dev.DeviceArray.from_numpy(va), dev.DeviceArray.from_numpy(vb))
        rk, rv = oracle.set_operation_by_key(op, a, b, va, vb)
        assert cnt == rk.size and np.array_equal(ko.numpy()[:cnt], rk) and np.array_equal(vo.numpy()[:cnt], rv), (op, seed)
        out, cnt = dev.set_operation(op, dev.DeviceArray.from_numpy(a), dev.DeviceArray.from_numpy(b))
        assert cnt == rk.size and np.array_equal(out.numpy()[:cnt], rk), (op, seed)


def test_set_operation_signed_zero_keeps_the_copy_of_the_named_side(dev, oracle):
    """-0.0 and +0.0 are equivalent keys with different bits: the kept copy is the one the
    reference's loop emits."""
    a = np.array([-1.0, -0.0, -0.0, 0.0, 2.0], np.float32)
    b = np.array([0.0, 0.0, -0.0, -0.0, 0.0, 3.0], np.float32)
    for op in OPS:
        out, cnt = dev.set_operation(op, dev.DeviceArray.from_numpy(a), dev.DeviceArray.from_numpy(b))
        ref = oracle.set_operation(op, a, b)
        assert cnt == ref.size and np.array_equal(out.numpy()[:cnt].view(np.uint32), ref.view(np.uint32)), op


def test_set_operation_large_properties(dev):
    """2 x 2^24 keys: sizes obey |A u B| + |A n B| = |A| + |B| and |A - B| + |A n B| = |A|,
    outputs are sorted, and union = merge of the difference pieces (checked by counts)."""
    n = 1 << 24
    a = np.sort((datagen.splitmix64(81, n) % np.uint64(n // 2)).astype(np.uint32))
    b = np.sort((datagen.splitmix64(82, n) % np.uint64(n // 2)).astype(np.uint32))
    da, db = dev.DeviceArray.from_numpy(a), dev.DeviceArray.from_numpy(b)
    sizes = {}
    for op in OPS:
        out, cnt = dev.set_operation(op, da, db)
        res = out.numpy()[:cnt]
        assert np.all(res[1:] >= res[:-1])
        sizes[op] = cnt
        if op == 1:
            # multiset intersection size from the two histograms
            ha, hb = np.bincount(a, minlength=n // 2), np.bincount(b, minlength=n // 2)
            assert cnt == int(np.minimum(ha, hb).sum())
            assert np.array_equal(np.bincount(res, minlength=n // 2), np.minimum(ha, hb))
    assert sizes[3] + sizes[1] == 2 * n
    assert sizes[0] + sizes[1] == n
    assert sizes[2] == sizes[3] - sizes[1]


def test_set_operation_rejects_bad_arguments(dev):
    d = dev.DeviceArray.from_numpy(np.zeros(4, np.int32))
    with pytest.raises(dev.ThrustAmdError):
        dev.set_operation(4, d, d)
    with pytest.raises(dev.ThrustAmdError):
        dev.set_operation(-1, d, d)
