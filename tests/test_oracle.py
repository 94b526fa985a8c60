"""CPU tests that pin the oracle (the C restatement of the reference's OMP / sequential
device system) -- no GPU involved.

Three independent anchors:
  1. the literal known-answer vectors of the reference's own unit tests
     (tests/golden/known_answers.json),
  2. outputs of the REAL reference on seeded inputs (tests/golden/small.npz, digests.json,
     written by tests/golden/make_fixtures.py from oracle/_ref), and live against
     oracle/_ref where that library is present,
  3. independent definitions: numpy cumsum modulo 2^k, np.sort(kind="stable"),
     boolean-mask filters, np.add.reduceat in float64, closed forms.
"""
import json
import os
import sys

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))

import cases  # noqa: E402
from oracle import cpu  # noqa: E402
from thrust_amd import datagen  # noqa: E402

KA = json.load(open(os.path.join(HERE, "golden", "known_answers.json")))
SMALL = np.load(os.path.join(HERE, "golden", "small.npz"))
DIGESTS = json.load(open(os.path.join(HERE, "golden", "digests.json")))

I32 = np.int32


# ---------------------------------------------------------------- 1. known answers
def test_known_reduce(oracle):
    for c in KA["reduce"]:
        assert oracle.reduce(np.array(c["in"], c["dtype"]), init=c["init"]) == c["out"]


def test_known_decompose(oracle):
    for c in KA["decompose"]:
        ranges = oracle.decompose(c["n"], c["granularity"], c["max_intervals"])
        assert [e - b for b, e in ranges] == c["sizes"]
        assert ranges[0][0] == 0 and ranges[-1][1] == c["n"]


def test_known_scans(oracle):
    for c in KA["inclusive_scan"]:
        assert oracle.inclusive_scan(np.array(c["in"], c["dtype"])).tolist() == c["out"]
    for c in KA["exclusive_scan"]:
        assert oracle.exclusive_scan(np.array(c["in"], c["dtype"]), c["init"]).tolist() == c["out"]


def test_known_sorts(oracle, oracle_seq):
    for o in (oracle, oracle_seq):
        for c in KA["sort"]:
            assert o.sort_keys(np.array(c["in"], c["dtype"])).tolist() == c["out"]
        for c in KA["sort_by_key"]:
            k, v = o.sort_pairs(np.array(c["keys"], I32), np.array(c["values"], I32))
            assert k.tolist() == c["keys_out"] and v.tolist() == c["values_out"]


def test_known_by_key_and_selection(oracle):
    for c in KA["reduce_by_key"]:
        k, v = oracle.reduce_by_key(np.array(c["keys"], I32), np.array(c["values"], I32))
        assert k.tolist() == c["keys_out"] and v.tolist() == c["values_out"]
    for c in KA["unique"]:
        assert oracle.unique(np.array(c["in"], I32)).tolist() == c["out"]
    for c in KA["unique_by_key"]:
        k, v = oracle.unique_by_key(np.array(c["keys"], I32), np.array(c["values"], I32))
        assert k.tolist() == c["keys_out"] and v.tolist() == c["values_out"]
    for c in KA["copy_if"]:
        assert oracle.copy_if(np.array(c["in"], I32), cpu.NONZERO).tolist() == c["out"]
    for c in KA["stable_partition"]:
        out, split = oracle.stable_partition(np.array(c["in"], I32), cpu.NONZERO,
                                             stencil=np.array(c["stencil_is_even"], I32))
        assert out.tolist() == c["out"] and split == c["split"]


def test_known_scan_by_key_count_inner_product(oracle):
    for c in KA["inclusive_scan_by_key"]:
        got = oracle.inclusive_scan_by_key(np.array(c["keys"], I32), np.array(c["values"], I32))
        assert got.tolist() == c["out"]
    for c in KA["exclusive_scan_by_key"]:
        got = oracle.exclusive_scan_by_key(np.array(c["keys"], I32), np.array(c["values"], I32), init=c["init"])
        assert got.tolist() == c["out"]
    codes = {"gt": cpu.GT, "eq": cpu.EQ}
    for c in KA["count_if"]:
        assert oracle.count_if(np.array(c["in"], I32), codes[c["cmp"]], c["threshold"]) == c["out"]
    for c in KA["inner_product"]:
        assert oracle.inner_product(np.array(c["a"], I32), np.array(c["b"], I32), init=c["init"]) == c["out"]


def test_known_transform_reduce_and_scans(oracle):
    un = {"identity": cpu.IDENTITY, "negate": cpu.NEGATE, "square": cpu.SQUARE}
    ops = {"plus": cpu.PLUS, "min": cpu.MIN, "max": cpu.MAX}
    for c in KA["transform_reduce"]:
        assert oracle.transform_reduce(np.array(c["in"], I32), un[c["unary"]], ops[c["op"]], c["init"]) == c["out"]
    for c in KA["transform_inclusive_scan"]:
        got = oracle.transform_inclusive_scan(np.array(c["in"], I32), un[c["unary"]], ops[c["op"]])
        assert got.tolist() == c["out"]
    for c in KA["transform_exclusive_scan"]:
        got = oracle.transform_exclusive_scan(np.array(c["in"], I32), un[c["unary"]], c["init"], ops[c["op"]])
        assert got.tolist() == c["out"]


def test_known_mixed_types(oracle):
    """testing/reduce.cu:98-129 and testing/scan.cu:236-297: which type accumulates."""
    for c in KA["reduce_mixed"]:
        init = np.dtype(c["init_dtype"]).type(c["init"])
        got = oracle.reduce_as(np.array(c["in"], c["in_dtype"]), init)
        assert got.dtype == init.dtype and got == c["out"], c["source"]
    for c in KA["scan_mixed"]:
        x = np.array(c["in"], c["in_dtype"])
        if c["kind"] == "inclusive":
            got = oracle.inclusive_scan_as(x, np.dtype(c["out_dtype"]))
        else:
            got = oracle.exclusive_scan_as(x, np.dtype(c["init_dtype"]).type(c["init"]), np.dtype(c["out_dtype"]))
        assert got.dtype == np.dtype(c["out_dtype"]) and got.tolist() == c["out"], c["source"]
    # conversions follow C's rules: truncation toward zero, wrap-around for narrower integers
    assert oracle.convert(np.array([-1.9, -0.5, 0.5, 1.9, 126.99], np.float64), np.int8).tolist() == [-1, 0, 0, 1, 126]
    assert oracle.convert(np.array([-1, 255, 256, 70000], np.int32), np.uint8).tolist() == [255, 255, 0, 112]
    assert oracle.convert(np.array([-1, 3], np.int8), np.uint64).tolist() == [2 ** 64 - 1, 3]
    assert oracle.convert(np.array([2 ** 24 + 1], np.int32), np.float32).tolist() == [float(2 ** 24)]


def test_known_comparison_sort(oracle):
    """testing/stable_sort.cu:49-90, stable_sort_by_key.cu:50-95: less_div_10 keeps the input order of equivalents."""
    kinds = {"less": cpu.CMP_SORT_LESS, "greater": cpu.CMP_SORT_GREATER, "less_div": cpu.CMP_SORT_LESS_DIV}
    for c in KA["comparison_sort"]:
        keys = np.array(c["keys"], I32)
        if "values" in c:
            k, v = oracle.comparison_sort(keys, np.array(c["values"], np.uint32), kinds[c["comparator"]], c["param"])
            assert k.tolist() == c["keys_out"] and v.tolist() == c["values_out"], c["source"]
        else:
            assert oracle.comparison_sort(keys, None, kinds[c["comparator"]], c["param"]).tolist() == c["keys_out"], c["source"]


def test_comparison_sort_against_numpy_stable_sort(oracle):
    """Stability fixes the answer: numpy's stable argsort of the comparator's key gives the same permutation."""
    for dtype in (np.int8, np.uint16, np.int32, np.uint64, np.float32, np.float64):
        for n in (0, 1, 31, 32, 33, 64, 65, 1000, 50001):
            x = ((datagen.splitmix64(71, n) % np.uint64(97)).astype(np.int64) - (0 if np.dtype(dtype).kind == "u" else 48)).astype(dtype)
            v = np.arange(n, dtype=np.uint32)
            k, w = oracle.comparison_sort(x, v, cpu.CMP_SORT_LESS)
            order = np.argsort(x, kind="stable")
            assert np.array_equal(w, order.astype(np.uint32)) and np.array_equal(k, x[order]), (dtype, n)
            k, w = oracle.comparison_sort(x, v, cpu.CMP_SORT_GREATER)
            order = np.argsort(-x.astype(np.float64), kind="stable")
            assert np.array_equal(w, order.astype(np.uint32)) and np.array_equal(k, x[order]), (dtype, n)
            k, w = oracle.comparison_sort(x, v, cpu.CMP_SORT_LESS_DIV, 10)
            order = np.argsort(np.trunc(x.astype(np.float64) / 10), kind="stable")  # C division truncates
            assert np.array_equal(w, order.astype(np.uint32)) and np.array_equal(k, x[order]), (dtype, n)
    # -0.0 and +0.0 are equivalent under operator< and keep their input order
    z = np.array([0.0, -0.0, 1.0, -0.0, 0.0, -1.0], np.float32)
    assert oracle.comparison_sort(z).tobytes() == np.array([-1.0, 0.0, -0.0, -0.0, 0.0, 1.0], np.float32).tobytes()


def test_known_set_operations(oracle):
    codes = {"difference": cpu.SET_DIFFERENCE, "intersection": cpu.SET_INTERSECTION,
             "symmetric_difference": cpu.SET_SYMMETRIC_DIFFERENCE, "union": cpu.SET_UNION}
    for c in KA["set_operation"]:
        got = oracle.set_operation(codes[c["op"]], np.array(c["a"], I32), np.array(c["b"], I32), c.get("descending", False))
        assert got.tolist() == c["out"], c["source"]
    for c in KA["set_operation_by_key"]:
        k, v = oracle.set_operation_by_key(codes[c["op"]], np.array(c["a_keys"], I32), np.array(c["b_keys"], I32),
                                           np.array(c["a_values"], np.uint32), np.array(c["b_values"], np.uint32),
                                           c.get("descending", False))
        assert k.tolist() == c["keys_out"] and v.tolist() == c["values_out"], c["source"]


def test_set_operations_against_multiset_definition(oracle):
    """Independent definition: with h_a, h_b the histograms of the two ranges, the result's
    histogram is max(h_a - h_b, 0), min, |h_a - h_b| and max; the result is sorted; and the
    by-key values name the side and the copies the two-pointer loop keeps (for a key with m
    copies in A and n in B: A's first min(m, n) for intersection, A's last m - n for
    difference, all of A then B's last n - m for union)."""
    n = 20000
    a = np.sort((datagen.splitmix64(21, n) % np.uint64(3000)).astype(np.int32))
    b = np.sort((datagen.splitmix64(22, n // 2) % np.uint64(3000)).astype(np.int32))
    ha, hb = np.bincount(a, minlength=3000), np.bincount(b, minlength=3000)
    want = {cpu.SET_DIFFERENCE: np.maximum(ha - hb, 0), cpu.SET_INTERSECTION: np.minimum(ha, hb),
            cpu.SET_SYMMETRIC_DIFFERENCE: np.abs(ha - hb), cpu.SET_UNION: np.maximum(ha, hb)}
    va, vb = np.arange(a.size, dtype=np.uint32), np.arange(b.size, dtype=np.uint32) + np.uint32(1 << 20)
    first_a = np.searchsorted(a, np.arange(3000))
    first_b = np.searchsorted(b, np.arange(3000))
    for op, hist in want.items():
        got = oracle.set_operation(op, a, b)
        assert np.all(got[1:] >= got[:-1]) and np.array_equal(np.bincount(got, minlength=3000), hist)
        k, v = oracle.set_operation_by_key(op, a, b, va, vb)
        assert np.array_equal(k, got)
        expect = []
        for x in range(3000):
            m, nn = int(ha[x]), int(hb[x])
            ia, ib = int(first_a[x]), int(first_b[x]) + (1 << 20)
            if op == cpu.SET_INTERSECTION:
                expect += range(ia, ia + min(m, nn))
            elif op == cpu.SET_DIFFERENCE:
                expect += range(ia + min(m, nn), ia + m)
            elif op == cpu.SET_UNION:
                expect += list(range(ia, ia + m)) + list(range(ib + min(m, nn), ib + nn))
            else:
                expect += list(range(ia + min(m, nn), ia + m)) + list(range(ib + min(m, nn), ib + nn))
        assert v.tolist() == expect, op
    # descending inputs mirror the ascending result
    ad, bd = a[::-1].copy(), b[::-1].copy()
    for op in want:
        assert np.array_equal(np.bincount(oracle.set_operation(op, ad, bd, True), minlength=3000), want[op])


def test_known_merges(oracle):
    for c in KA["merge"]:
        assert oracle.merge(np.array(c["a"], I32), np.array(c["b"], I32)).tolist() == c["out"]
    for c in KA["merge_by_key"]:
        k, v = oracle.merge_by_key(np.array(c["a_keys"], I32), np.array(c["b_keys"], I32),
                                   np.array(c["a_values"], I32), np.array(c["b_values"], I32))
        assert k.tolist() == c["keys_out"] and v.tolist() == c["values_out"]


# ---------------------------------------------------------------- 2. the real reference
def _bytes_equal(a, b):
    return np.array_equal(np.ascontiguousarray(a).view(np.uint8), np.ascontiguousarray(b).view(np.uint8))


@pytest.mark.parametrize("case", sorted(cases.CASES))
def test_oracle_reproduces_reference_fixtures(oracle, oracle_seq, case):
    impl = oracle_seq if case == "c2" else oracle
    got = cases.CASES[case](impl, cases.SMALL[case])
    assert got, case
    for name, arr in got.items():
        assert _bytes_equal(arr, SMALL[name]), name


@pytest.mark.parametrize("case", sorted(cases.CASES))
def test_oracle_reproduces_reference_digests(oracle, oracle_seq, case):
    impl = oracle_seq if case == "c2" else oracle
    got = cases.CASES[case](impl, cases.LARGE[case])
    for name, arr in got.items():
        assert cases.digest(arr) == DIGESTS["sha256"][name], name


@pytest.mark.skipif(not (cpu.ref_available("omp") and cpu.ref_available("cpp")),
                    reason="oracle/_ref is built only where the reference tree is present")
def test_oracle_matches_live_reference_on_ragged_sizes(oracle, oracle_seq):
    omp, cpp = cpu.Reference("omp"), cpu.Reference("cpp")
    for n in [0, 1, 2, 7, 8, 9, 63, 1000, 4099, 70001]:
        x = (datagen.splitmix64(3, n) % np.uint64(1001)).astype(np.int32)
        assert oracle.reduce(x, init=5) == omp.reduce(x, init=5) == cpp.reduce(x, init=5)
        assert np.array_equal(oracle.inclusive_scan(x), omp.inclusive_scan(x))
        assert np.array_equal(oracle.exclusive_scan(x, 3), cpp.exclusive_scan(x, 3))
        for dt in (np.uint32, np.int64, np.float32, np.float64, np.uint8, np.int16):
            k = (datagen.splitmix64(5, n) >> np.uint64(11)).astype(dt)
            if np.dtype(dt).kind == "f":
                k = (k / dt(3.0) - dt(1e5)).astype(dt)
                if n > 4:
                    k[1], k[3] = dt(-0.0), dt(0.0)
            assert _bytes_equal(oracle_seq.sort_keys(k), cpp.sort_keys(k)), (dt, n)
            assert _bytes_equal(oracle_seq.sort_keys(k, True), cpp.sort_keys(k, True)), (dt, n)
            v = np.arange(n, dtype=np.uint32)
            kk = (k.astype(np.float64) % 7).astype(dt)
            a, b = oracle.sort_pairs(kk, v), omp.sort_pairs(kk, v)
            assert _bytes_equal(a[0], b[0]) and np.array_equal(a[1], b[1]), (dt, n)
            a, b = oracle.sort_pairs(kk, v, True), omp.sort_pairs(kk, v, True)
            assert _bytes_equal(a[0], b[0]) and np.array_equal(a[1], b[1]), (dt, n)
        for dt in (np.int8, np.uint16, np.int32, np.uint64, np.float32, np.float64):
            t = ((datagen.splitmix64(15, n) % np.uint64(200)).astype(np.int64) - 100).astype(dt)
            for un in (cpu.NEGATE, cpu.SQUARE):
                for op in (cpu.PLUS, cpu.MIN, cpu.MAX):
                    assert _bytes_equal(oracle.transform_reduce(t, un, op, 3), omp.transform_reduce(t, un, op, 3)), (dt, n)
                    assert _bytes_equal(oracle.transform_inclusive_scan(t, un, op), cpp.transform_inclusive_scan(t, un, op))
                    assert _bytes_equal(oracle.transform_exclusive_scan(t, un, 3, op), omp.transform_exclusive_scan(t, un, 3, op))
        for dt in (np.int32, np.uint64, np.float32):
            sa = np.sort((datagen.splitmix64(17, n) % np.uint64(n // 3 + 2)).astype(dt))
            sb = np.sort((datagen.splitmix64(19, n // 2 + 1) % np.uint64(n // 3 + 2)).astype(dt))
            wa, wb = np.arange(sa.size, dtype=np.uint32), np.arange(sb.size, dtype=np.uint32) + np.uint32(1 << 30)
            for op in range(4):
                assert _bytes_equal(oracle.set_operation(op, sa, sb), omp.set_operation(op, sa, sb)), (dt, n, op)
                assert _bytes_equal(oracle.set_operation(op, sa[::-1].copy(), sb[::-1].copy(), True),
                                    cpp.set_operation(op, sa[::-1].copy(), sb[::-1].copy(), True)), (dt, n, op)
                x, y = oracle.set_operation_by_key(op, sa, sb, wa, wb), omp.set_operation_by_key(op, sa, sb, wa, wb)
                assert _bytes_equal(x[0], y[0]) and np.array_equal(x[1], y[1]), (dt, n, op)
        # comparison sort: user-defined comparators take the reference's merge sort
        cx = (datagen.splitmix64(31, n) % np.uint64(199)).astype(np.int32) - np.int32(99)
        cf = np.where(datagen.u01(33, n) < 0.1, np.float32(-0.0), cx.astype(np.float32) / 4).astype(np.float32)
        cv = np.arange(n, dtype=np.uint32)
        for ref in (omp, cpp):
            for comparator, param in ((cpu.CMP_SORT_LESS, 0), (cpu.CMP_SORT_GREATER, 0), (cpu.CMP_SORT_LESS_DIV, 10)):
                for keys in (cx, cf, cx.astype(np.int8), cx.astype(np.int64)):
                    x, y = oracle.comparison_sort(keys, cv, comparator, param), ref.comparison_sort(keys, cv, comparator, param)
                    assert _bytes_equal(x[0], y[0]) and np.array_equal(x[1], y[1]), (n, comparator, keys.dtype)
                assert _bytes_equal(oracle.comparison_sort(cf, None, comparator, param), ref.comparison_sort(cf, None, comparator, param))
        # mixed element types: the reference's own type deduction against the restated rule
        fx = (datagen.u01(23, n) * 64 - 32).astype(np.float32)
        ix = (datagen.splitmix64(29, n) % np.uint64(2001)).astype(np.int32) - np.int32(1000)
        for ref in (omp, cpp):
            assert oracle.reduce_as(fx, np.int32(7)) == ref.reduce_as(fx, np.int32(7)), n
            assert _bytes_equal(oracle.exclusive_scan_as(ix, np.int32(3), np.float32), ref.exclusive_scan_as(ix, np.int32(3), np.float32))
            assert _bytes_equal(oracle.inclusive_scan_as(ix, np.float32), ref.inclusive_scan_as(ix, np.float32))
            for dt_in, dt_out in ((np.float32, np.int32), (np.int64, np.uint8), (np.uint16, np.float64), (np.float64, np.float32)):
                src = (fx.astype(np.float64) * 1.37).astype(dt_in) if np.dtype(dt_in).kind == "f" else ix.astype(dt_in)
                if np.dtype(dt_out).kind != "f" and np.dtype(dt_in).kind == "f":
                    src = np.clip(src, -1e6, 1e6).astype(dt_in)
                assert _bytes_equal(oracle.convert(src, dt_out), ref.convert(src, dt_out)), (dt_in, dt_out)
        # float accumulators: one thread, so that the order of additions is the sequential one
        assert oracle_seq.reduce_as(ix, np.float32(0.5)) == cpp.reduce_as(ix, np.float32(0.5)), n
        assert _bytes_equal(oracle_seq.inclusive_scan_as(fx, np.int32), cpp.inclusive_scan_as(fx, np.int32))
        assert _bytes_equal(oracle_seq.exclusive_scan_as(fx, np.float32(5.5), np.int32), cpp.exclusive_scan_as(fx, np.float32(5.5), np.int32))
        assert _bytes_equal(oracle_seq.exclusive_scan_as(ix, np.float32(5.5), np.float32), cpp.exclusive_scan_as(ix, np.float32(5.5), np.float32))
        keys = np.sort((datagen.splitmix64(7, n) % np.uint64(50)).astype(np.int32))
        vals = datagen.u01(9, n)
        a, b = oracle.reduce_by_key(keys, vals), omp.reduce_by_key(keys, vals)
        assert np.array_equal(a[0], b[0]) and _bytes_equal(a[1], b[1])
        for op in (cpu.MIN, cpu.MAX):
            a, b = oracle.reduce_by_key(keys, vals, op), cpp.reduce_by_key(keys, vals, op)
            assert np.array_equal(a[0], b[0]) and _bytes_equal(a[1], b[1])
        a, b = oracle.unique_by_key(keys, vals), omp.unique_by_key(keys, vals)
        assert np.array_equal(a[0], b[0]) and _bytes_equal(a[1], b[1])
        assert np.array_equal(oracle.unique(keys), cpp.unique(keys))
        for cmp in range(6):
            assert _bytes_equal(oracle.copy_if(vals, cmp, 0.3), omp.copy_if(vals, cmp, 0.3))
        assert _bytes_equal(oracle.copy_if(vals, cpu.GT, 10, stencil=keys), omp.copy_if(vals, cpu.GT, 10, stencil=keys))
        a, b = oracle.stable_partition(vals, cpu.LT, 0.5), omp.stable_partition(vals, cpu.LT, 0.5)
        assert a[1] == b[1] and _bytes_equal(a[0], b[0])
        a, b = oracle.partition_copy(vals, cpu.LT, 0.5), cpp.partition_copy(vals, cpu.LT, 0.5)
        assert _bytes_equal(a[0], b[0]) and _bytes_equal(a[1], b[1])
        kb = np.sort((datagen.splitmix64(11, n // 2 + 1) % np.uint64(50)).astype(np.int32))
        va, vb = np.arange(n, dtype=np.uint64), np.arange(kb.size, dtype=np.uint64) + 10 ** 9
        a, b = oracle.merge_by_key(keys, kb, va, vb), omp.merge_by_key(keys, kb, va, vb)
        assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])


# ---------------------------------------------------------------- 3. independent definitions
def test_reduce_and_scan_are_sums_modulo_2k(oracle):
    for dt, bits in ((np.int8, 8), (np.uint16, 16), (np.int32, 32), (np.uint32, 32), (np.int64, 64)):
        x = (datagen.splitmix64(13, 100003) >> np.uint64(3)).astype(dt)
        exact = [int(v) for v in x]
        total = sum(exact)
        assert (int(oracle.reduce(x)) - total) % (1 << bits) == 0
        run, ok = 0, True
        scan = oracle.inclusive_scan(x)
        for i in (0, 1, 999, 50000, 100002):
            run = sum(exact[: i + 1])
            ok = ok and (int(scan[i]) - run) % (1 << bits) == 0
        assert ok
        ex = oracle.exclusive_scan(x, 9)
        assert int(ex[0]) == 9 and (int(ex[-1]) - (9 + total - exact[-1])) % (1 << bits) == 0


def test_reduce_is_independent_of_chunk_count_for_integers():
    x = datagen.c1_int32(100000)
    vals = {cpu.Oracle(nthreads=p).reduce(x) for p in (1, 2, 3, 7, 8, 64)}
    assert len(vals) == 1 and int(vals.pop()) == int(np.sum(x.astype(np.int64)))


def test_sort_against_numpy_stable_sort(oracle, oracle_seq):
    n = 200003
    k = datagen.c2_uint32(n)
    assert np.array_equal(oracle.sort_keys(k), np.sort(k, kind="stable"))
    ks = (k % np.uint32(100)).astype(np.uint32)
    v = np.arange(n, dtype=np.uint32)
    order = np.argsort(ks, kind="stable")
    a = oracle.sort_pairs(ks, v)
    assert np.array_equal(a[0], ks[order]) and np.array_equal(a[1], v[order])
    f = datagen.c2_float32(n)
    out = oracle_seq.sort_keys(f)
    u = out.view(np.uint32)
    enc = u ^ np.where(u >> 31, np.uint32(0xFFFFFFFF), np.uint32(0x80000000))
    assert np.all(enc[:-1] <= enc[1:])  # total order on the encoded bits: -0.0 before +0.0
    assert np.array_equal(np.sort(f), np.sort(out))


def test_float_sort_signed_zero_layout_depends_on_thread_count():
    """Why the parity comparator for float sorts is the sequential system: with several
    threads the merges compare with operator<, for which -0.0 == +0.0."""
    f = datagen.c2_float32(1 << 16)
    seq = cpu.Oracle(nthreads=1).sort_keys(f).view(np.uint32)
    par = cpu.Oracle(nthreads=8).sort_keys(f).view(np.uint32)
    assert np.array_equal(np.sort(seq), np.sort(par))  # same multiset of bit patterns
    assert np.array_equal(seq.view(np.float32), par.view(np.float32))  # equal as values


def test_selection_against_boolean_masks(oracle):
    x = datagen.c5_float32(100003)
    for t in (0.5, 0.05):
        m = x < np.float32(t)
        assert np.array_equal(oracle.copy_if(x, cpu.LT, t), x[m])
        out, split = oracle.stable_partition(x, cpu.LT, t)
        assert split == m.sum() and np.array_equal(out, np.r_[x[m], x[~m]])


def test_by_key_against_reduceat(oracle):
    k, v = datagen.c4_segments(100003, 8)
    starts = np.flatnonzero(np.r_[True, k[1:] != k[:-1]])
    ko, vo = oracle.reduce_by_key(k, v)
    assert np.array_equal(ko, k[starts])
    ref64 = np.add.reduceat(v.astype(np.float64), starts)
    assert np.max(np.abs(vo - ref64) / ref64) < 1e-5
    iv = (v * 1000).astype(np.int32)
    assert np.array_equal(oracle.reduce_by_key(k, iv)[1], np.add.reduceat(iv, starts))
    uk, uv = oracle.unique_by_key(k, v)
    assert np.array_equal(uk, k[starts]) and np.array_equal(uv, v[starts])


def test_merge_against_stable_sort_of_concatenation(oracle):
    (ka, va), (kb, vb) = datagen.c5_merge_inputs(50001)
    ka, kb = ka % np.uint32(1000), kb % np.uint32(1000)
    ka.sort(), kb.sort()
    ko, vo = oracle.merge_by_key(ka, kb, va, vb)
    order = np.argsort(np.r_[ka, kb], kind="stable")
    assert np.array_equal(ko, np.r_[ka, kb][order]) and np.array_equal(vo, np.r_[va, vb][order])


def test_scan_by_key_count_inner_product_against_numpy(oracle):
    """Independent definitions: per-segment cumulative sums (float64 / modulo 2^32), boolean
    masks, and the dot product modulo 2^k."""
    n = 100003
    k, v = datagen.c4_segments(n, 8)
    iv = (v * 1000).astype(np.int32)
    head = np.r_[True, k[1:] != k[:-1]]
    starts = np.flatnonzero(head)
    seg = np.cumsum(head) - 1
    c = np.cumsum(iv.astype(np.int64))
    incl = c - np.r_[0, c[:-1]][starts][seg]
    assert np.array_equal(oracle.inclusive_scan_by_key(k, iv), incl.astype(np.int32))
    assert np.array_equal(oracle.exclusive_scan_by_key(k, iv, init=9), (incl - iv + 9).astype(np.int32))
    # min / max: running extrema restart at every head
    mx = oracle.inclusive_scan_by_key(k, iv, op=cpu.MAX)
    assert np.array_equal(mx[starts], iv[starts]) and np.all(mx >= iv)
    assert np.array_equal(np.maximum.reduceat(iv, starts), mx[np.r_[starts[1:] - 1, n - 1]])
    x = datagen.c1_int32(n)
    for cmp, mask in ((cpu.LT, x < 500), (cpu.GE, x >= 500), (cpu.EQ, x == 500), (cpu.NONZERO, x != 0)):
        assert oracle.count_if(x, cmp, 500) == int(mask.sum())
    for dtype in (np.int8, np.uint16, np.int32, np.uint64):
        a = (datagen.splitmix64(1, n) >> np.uint64(5)).astype(dtype)
        b = (datagen.splitmix64(2, n) >> np.uint64(11)).astype(dtype)
        bits = 8 * np.dtype(dtype).itemsize
        exact = (sum(int(p) * int(q) for p, q in zip(a[:2000].tolist(), b[:2000].tolist())) + 3) % (1 << bits)
        got = int(oracle.inner_product(a[:2000], b[:2000], init=3)) % (1 << bits)
        assert got == exact, dtype
    # transform_reduce / transform scans: negate and square against numpy, modulo 2^bits
    for dtype in (np.int8, np.uint16, np.int32, np.uint64):
        bits = 8 * np.dtype(dtype).itemsize
        a = (datagen.splitmix64(4, 3000) >> np.uint64(9)).astype(dtype)
        ints = [int(v) for v in a]
        assert (int(oracle.transform_reduce(a, cpu.SQUARE, init=1)) - (sum(v * v for v in ints) + 1)) % (1 << bits) == 0
        assert (int(oracle.transform_reduce(a, cpu.NEGATE, init=1)) - (1 - sum(ints))) % (1 << bits) == 0
        sq = np.cumsum(np.array([(v * v) % (1 << bits) for v in ints], dtype=object))
        got = oracle.transform_inclusive_scan(a, cpu.SQUARE)
        assert all((int(g) - int(e)) % (1 << bits) == 0 for g, e in zip(got[::97], sq[::97]))
        ex = oracle.transform_exclusive_scan(a, cpu.NEGATE, init=7)
        assert int(ex[0]) % (1 << bits) == 7 and (int(ex[-1]) - (7 - sum(ints[:-1]))) % (1 << bits) == 0
    g = datagen.u01(8, 5000) - 0.5
    assert np.array_equal(oracle.transform_inclusive_scan(g, cpu.NEGATE, cpu.MAX), np.maximum.accumulate(-g))
    assert oracle.transform_reduce(g, cpu.SQUARE, cpu.MIN, init=9.0) == np.min(g * g)
    f = datagen.u01(7, n)
    assert abs(float(oracle.inner_product(f, f, init=1.0)) - (float(np.dot(f.astype(np.float64), f)) + 1.0)) < 1e-3 * n * 1e-4
