"""The benchmark configurations beside the headline one: each is run on the device at its own
size, its result is verified there against an independent torch computation, and the whole
call (every kernel it launches, launch gaps included) is timed with events on the launch
stream (three warm-ups, then the median and the minimum of 20 calls).  bench.py imports this module and
prints the rows inside its JSON line.

  C2  sort of 2^28 float32 keys (1 % of +-0.0 and denormals)
  C3  stable sort_by_key of 2^27 uint64 keys + uint32 values: full range / low 16 bits / 90 % one key
  C4  reduce_by_key, unique_by_key and unique over 2^28 (int32 key, float32 value), mean run 8 / 1000
  C5  copy_if and stable_partition of 2^28 float32 at 50 % / 5 % selectivity,
      merge_by_key and merge of two sorted ranges of 2^27 uint32 (+ uint32 values)
and the entry points beside the named path (rows "next_*"):
  C6  count_if, inner_product, transform_reduce, transform_exclusive_scan over 2^28, inclusive_scan_by_key
      over the C4 input with mean run 8
  C7  set_union and set_intersection of the two sorted C5 ranges
  C8  the comparison sort (merge sort) of 2^28 uint32 keys and of 2^27 uint64 keys with uint32 values

Bytes are the algorithmic ones of each call (what must be read and written once).
"""
import numpy as np

from . import datagen_device as gen

HBM_PEAK_GBS = 8000.0


def _dev(capi, torch, t, code):
    items = t.numel() * t.element_size() // np.dtype(capi.NP_DTYPES[code]).itemsize
    return capi.DeviceArray(items, code, t.view(torch.uint8))


def _hold_device(torch):
    """Keeps the device busy for a few hundred microseconds without touching memory, so that the
    host can enqueue the whole call before the opening event is reached.  (A large fill did the
    same job but left a gigabyte of dirty cache lines whose write-back ran into the timed call:
    30-40 us on every row, 60 us on the read-only ones.)"""
    torch.cuda._sleep(800_000)


def _time_calls(torch, fn, reps, setup=None):
    """Median and minimum device time of fn() in ms; setup() runs before each call, untimed.
    fn must not synchronise."""
    for _ in range(3):  # the first call sizes the temporary storage; three warm-ups in all
        if setup:
            setup()
        fn()
    torch.cuda.synchronize()
    times = []
    for _ in range(reps):
        if setup:
            setup()
        _hold_device(torch)
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        fn()
        b.record()
        b.synchronize()
        times.append(a.elapsed_time(b))
    times.sort()
    return times[len(times) // 2], times[0]


def _row(ms_med, ms_min, nbytes, **extra):
    gbs = nbytes / ms_med / 1e6
    row = {"ms": round(ms_med, 4), "ms_min": round(ms_min, 4), "GBps": round(gbs, 1),
           "pct_of_peak": round(gbs / HBM_PEAK_GBS * 100, 2), "bytes": int(nbytes), "verified": True}
    row.update(extra)
    return row


def _fail(what):
    raise SystemExit(f"bench: {what} failed its result check")


def run_c2_float(torch, capi, reps):
    n = 1 << 28
    f = gen.c2_float32(torch, n)
    src, work, t = _dev(capi, torch, f, capi.F32), capi.DeviceArray(n, capi.F32), capi.Temp()
    med, mn = _time_calls(torch, lambda: capi.sort_keys(work, temp=t), reps,
                          setup=lambda: work.storage.copy_(src.storage))
    out = work.storage.view(torch.int32)
    # radix order of floats: flip all bits of negatives, the sign bit of the others
    enc = lambda b: torch.where(b < 0, ~b, b ^ (-(1 << 31))).to(torch.int64) & 0xFFFFFFFF
    e = enc(out)
    if not bool((e[1:] >= e[:-1]).all().item()):
        _fail("C2 float32 sort (order)")
    if int(e.sum().item()) != int(enc(f.view(torch.int32)).sum().item()):
        _fail("C2 float32 sort (checksum)")
    return {"c2_sort_f32_2p28": _row(med, mn, 36 * n, Gkeys_per_s=round(n / med / 1e6, 2), model="36 B/key")}


def run_c3(torch, capi, reps):
    m = 1 << 27
    rows = {}
    for kind in ("full", "low16", "skew90"):
        keys = gen.c3_uint64(torch, m, kind)
        vals = torch.arange(m, dtype=torch.int32, device="cuda")
        sk, sv = _dev(capi, torch, keys, capi.U64), _dev(capi, torch, vals, capi.U32)
        wk, wv, t = capi.DeviceArray(m, capi.U64), capi.DeviceArray(m, capi.U32), capi.Temp()

        def setup():
            wk.storage.copy_(sk.storage)
            wv.storage.copy_(sv.storage)
        med, mn = _time_calls(torch, lambda: capi.sort_pairs(wk, wv, temp=t), reps, setup=setup)
        ko = wk.storage.view(torch.int64)
        vo = wv.storage.view(torch.int32).to(torch.int64)
        o = ko ^ (-(1 << 63))
        same = ko[1:] == ko[:-1]
        ok = bool((o[1:] >= o[:-1]).all().item()) and bool((keys[vo] == ko).all().item()) \
            and bool((vo[1:][same] > vo[:-1][same]).all().item())
        if not ok:
            _fail(f"C3 sort_by_key {kind}")
        # passes over a digit that is the same in every key move nothing (the reference's sequential radix
        # sort skips them too): the bytes of the call are the histogram read and the passes that run
        passes_run = sum(1 for p in range(8) if int(((keys >> (8 * p)) & 0xFF).min().item())
                         != int(((keys >> (8 * p)) & 0xFF).max().item()))
        rows[f"c3_sort_by_key_u64_u32_2p27_{kind}"] = _row(
            med, mn, (8 + 24 * passes_run) * m, Gpairs_per_s=round(m / med / 1e6, 2), passes_run=passes_run,
            model="8 B/pair histogram read + 24 B/pair per pass that runs (all 8: 200 B/pair)")
        del keys, vals, sk, sv, wk, wv, t, ko, vo, o, same
    return rows


def run_c4(torch, capi, reps):
    n = 1 << 28
    rows = {}
    for mean in (8, 1000):
        keys, vals = gen.c4_segments(torch, n, mean)
        runs = int(keys[-1].item()) + 1
        dk, dv = _dev(capi, torch, keys, capi.I32), _dev(capi, torch, vals, capi.F32)
        ko, vo, t = capi.DeviceArray(n, capi.I32), capi.DeviceArray(n, capi.F32), capi.Temp()
        starts = torch.searchsorted(keys, torch.arange(runs, dtype=torch.int32, device="cuda"))
        want_keys = torch.arange(runs, dtype=torch.int32, device="cuda")

        res = {}
        med, mn = _time_calls(torch, lambda: res.update(r=capi.reduce_by_key(dk, dv, temp=t, keys_out=ko, values_out=vo, read_count=False)), reps)
        cnt = int(res["r"][-1].numpy()[0])
        sums = torch.zeros(runs, dtype=torch.float64, device="cuda").index_add_(0, keys.to(torch.int64), vals.to(torch.float64))
        got = vo.storage.view(torch.float32)[:runs].to(torch.float64)
        rel = ((got - sums).abs() / sums.abs().clamp_min(1e-30)).max().item()
        if cnt != runs or not torch.equal(ko.storage.view(torch.int32)[:runs], want_keys) or rel > 1e-5:
            _fail(f"C4 reduce_by_key mean {mean} (count {cnt} vs {runs}, rel {rel:.2e})")
        rows[f"c4_reduce_by_key_mean{mean}"] = _row(med, mn, 8 * n + 8 * runs, runs=runs, max_rel_err_vs_f64=float(f"{rel:.3e}"))

        med, mn = _time_calls(torch, lambda: res.update(r=capi.unique_by_key(dk, dv, keys_out=ko, values_out=vo, temp=t, read_count=False)), reps)
        cnt = int(res["r"][-1].numpy()[0])
        if cnt != runs or not torch.equal(ko.storage.view(torch.int32)[:runs], want_keys) \
                or not torch.equal(vo.storage.view(torch.float32)[:runs], vals[starts]):
            _fail(f"C4 unique_by_key mean {mean}")
        rows[f"c4_unique_by_key_mean{mean}"] = _row(med, mn, 8 * n + 8 * runs, runs=runs)

        med, mn = _time_calls(torch, lambda: res.update(r=capi.unique(dk, out=ko, temp=t, read_count=False)), reps)
        cnt = int(res["r"][-1].numpy()[0])
        if cnt != runs or not torch.equal(ko.storage.view(torch.int32)[:runs], want_keys):
            _fail(f"C4 unique mean {mean}")
        rows[f"c4_unique_keys_mean{mean}"] = _row(med, mn, 4 * n + 4 * runs, runs=runs)
        del keys, vals, dk, dv, ko, vo, t, starts, want_keys, sums, got
    return rows


def run_c5(torch, capi, reps):
    n = 1 << 28
    rows = {}
    x = gen.c5_float32(torch, n)
    dx, out, work = _dev(capi, torch, x, capi.F32), capi.DeviceArray(n, capi.F32), capi.DeviceArray(n, capi.F32)
    t, tp = capi.Temp(), capi.Temp()
    for thr, tag in ((0.5, "50pct"), (0.05, "5pct")):
        thr32 = float(np.float32(thr))
        mask = x < thr32
        want_true = x[mask]
        cnt_want = want_true.numel()
        res = {}
        med, mn = _time_calls(torch, lambda: res.update(r=capi.copy_if(dx, capi.LT, thr, out=out, temp=t, read_count=False)), reps)
        cnt = int(res["r"][-1].numpy()[0])
        if cnt != cnt_want or not torch.equal(out.storage.view(torch.float32)[:cnt], want_true):
            _fail(f"C5 copy_if {tag}")
        rows[f"c5_copy_if_{tag}"] = _row(med, mn, 4 * n + 4 * cnt, selected=cnt)

        med, mn = _time_calls(torch, lambda: res.update(r=(capi.stable_partition(work, capi.LT, thr, temp=tp, read_count=False),)), reps,
                              setup=lambda: work.storage.copy_(dx.storage))
        cnt = int(res["r"][-1].numpy()[0])
        got = work.storage.view(torch.float32)
        if cnt != cnt_want or not torch.equal(got[:cnt], want_true) or not torch.equal(got[cnt:], x[~mask]):
            _fail(f"C5 stable_partition {tag}")
        # in place the smaller side is parked in temporary storage and copied back: 8 bytes more per parked element
        moved = 8 * n + 8 * min(cnt, n - cnt)
        rows[f"c5_stable_partition_{tag}"] = _row(
            med, mn, 8 * n, selected=cnt, bytes_moved=int(moved),
            pct_of_peak_moved=round(moved / med / 1e6 / HBM_PEAK_GBS * 100, 2))
        del mask, want_true, got
    del x, dx, out, work, t, tp

    m = 1 << 27
    (ka, va), (kb, vb) = gen.c5_merge_inputs(torch, m)
    vb = vb + m  # payloads of the second range are told apart from the first's
    a = [_dev(capi, torch, z, capi.U32) for z in (ka, kb, va, vb)]
    ko, vo, t, t2 = capi.DeviceArray(2 * m, capi.U32), capi.DeviceArray(2 * m, capi.U32), capi.Temp(), capi.Temp()
    # a stable sort of (first range, second range) is the merge with ties from the first range first
    both = torch.cat([ka, kb]).to(torch.int64) & 0xFFFFFFFF
    want_k, order = torch.sort(both, stable=True)
    want_v = torch.cat([va, vb])[order]
    med, mn = _time_calls(torch, lambda: capi.merge_by_key(*a, temp=t, keys_out=ko, values_out=vo), reps)
    if not torch.equal(ko.storage.view(torch.int32).to(torch.int64) & 0xFFFFFFFF, want_k) \
            or not torch.equal(vo.storage.view(torch.int32), want_v):
        _fail("C5 merge_by_key")
    rows["c5_merge_by_key_2x2p27"] = _row(med, mn, 16 * 2 * m)
    med, mn = _time_calls(torch, lambda: capi.merge(a[0], a[1], out=ko, temp=t2), reps)
    if not torch.equal(ko.storage.view(torch.int32).to(torch.int64) & 0xFFFFFFFF, want_k):
        _fail("C5 merge")
    rows["c5_merge_2x2p27"] = _row(med, mn, 8 * 2 * m)
    return rows


def run_c6(torch, capi, reps):
    n = 1 << 28
    rows = {}
    xi = gen.c1_int32(torch, n)
    di, t = _dev(capi, torch, xi, capi.I32), capi.Temp()
    res = {}
    med, mn = _time_calls(torch, lambda: res.update(r=capi.count_if(di, capi.LT, 500, temp=t, read_count=False)), reps)
    if int(res["r"].numpy()[0]) != int((xi < 500).sum().item()):
        _fail("C6 count_if")
    rows["next_c6_count_if_i32"] = _row(med, mn, 4 * n)
    oi, t2 = capi.DeviceArray(n, capi.I32), capi.Temp()
    med, mn = _time_calls(torch, lambda: capi.transform_exclusive_scan(di, capi.SQUARE, 0, out=oi, temp=t2), reps)
    sq = xi.to(torch.int64)
    sq = sq * sq
    want = torch.cumsum(sq, 0) - sq  # exclusive; values stay far below 2^63
    if not torch.equal(oi.storage.view(torch.int32).to(torch.int64) & 0xFFFFFFFF, want & 0xFFFFFFFF):
        _fail("C6 transform_exclusive_scan")
    rows["next_c6_transform_exclusive_scan_i32_square"] = _row(med, mn, 8 * n)
    del xi, di, oi, sq, want

    xf, yf = gen.c5_float32(torch, n), gen.c5_float32(torch, n, seed=7)
    df, dy, o1, t = _dev(capi, torch, xf, capi.F32), _dev(capi, torch, yf, capi.F32), capi.DeviceArray(1, capi.F32), capi.Temp()
    exact = float((xf.to(torch.float64) * yf.to(torch.float64)).sum().item())
    med, mn = _time_calls(torch, lambda: capi.inner_product(df, dy, 0, temp=t, out=o1), reps)
    if abs(float(o1.numpy()[0]) - exact) > 1e-5 * exact:
        _fail("C6 inner_product")
    rows["next_c6_inner_product_f32"] = _row(med, mn, 8 * n)
    del yf, dy
    exact = float((xf.to(torch.float64) ** 2).sum().item())
    t = capi.Temp()
    med, mn = _time_calls(torch, lambda: capi.transform_reduce(df, capi.SQUARE, capi.PLUS, 0, temp=t, out=o1), reps)
    if abs(float(o1.numpy()[0]) - exact) > 1e-5 * exact:
        _fail("C6 transform_reduce")
    rows["next_c6_transform_reduce_f32_square"] = _row(med, mn, 4 * n)
    del xf, df

    keys, vals = gen.c4_segments(torch, n, 8)
    dk, dv = _dev(capi, torch, keys, capi.I32), _dev(capi, torch, vals, capi.F32)
    out, t = capi.DeviceArray(n, capi.F32), capi.Temp()
    med, mn = _time_calls(torch, lambda: capi.inclusive_scan_by_key(dk, dv, out=out, temp=t), reps)
    # float64 running sums that start over at every run: the cumulative sum minus its value before the run
    cs = torch.cumsum(vals.to(torch.float64), 0)
    runs = int(keys[-1].item()) + 1
    starts = torch.searchsorted(keys, torch.arange(runs, dtype=torch.int32, device="cuda"))
    before = torch.where(starts > 0, cs[(starts - 1).clamp_min(0)], torch.zeros_like(cs[:1]))
    want = cs - before[keys.to(torch.int64)]
    if float((out.storage.view(torch.float32).to(torch.float64) - want).abs().max().item()) > 1e-4:
        _fail("C6 inclusive_scan_by_key")
    rows["next_c6_inclusive_scan_by_key_mean8"] = _row(med, mn, 12 * n)
    return rows


def _multiplicities(torch, sorted_u, uniq):
    return torch.searchsorted(sorted_u, uniq, right=True) - torch.searchsorted(sorted_u, uniq)


def run_c7(torch, capi, reps):
    m = 1 << 27
    (ka, _), (kb, _) = gen.c5_merge_inputs(torch, m)
    a, b = _dev(capi, torch, ka, capi.U32), _dev(capi, torch, kb, capi.U32)
    out = capi.DeviceArray(2 * m, capi.U32)
    ua, ub = ka.to(torch.int64) & 0xFFFFFFFF, kb.to(torch.int64) & 0xFFFFFFFF
    uniq = torch.unique(torch.cat([ua, ub]))
    ca, cb = _multiplicities(torch, ua, uniq), _multiplicities(torch, ub, uniq)
    rows = {}
    for op, name, want in ((capi.SET_UNION, "set_union", torch.maximum(ca, cb)),
                           (capi.SET_INTERSECTION, "set_intersection", torch.minimum(ca, cb))):
        t, res = capi.Temp(), {}
        med, mn = _time_calls(torch, lambda: res.update(r=capi.set_operation(op, a, b, out=out, temp=t, read_count=False)), reps)
        cnt = int(res["r"][-1].numpy()[0])
        got = out.storage.view(torch.int32)[:cnt].to(torch.int64) & 0xFFFFFFFF
        # the multiset definition: every key as often as the rule says, in order
        if cnt != int(want.sum().item()) or not bool((got[1:] >= got[:-1]).all().item()) \
                or not torch.equal(_multiplicities(torch, got, uniq), want):
            _fail(f"C7 {name}")
        rows[f"next_c7_{name}_2x2p27"] = _row(med, mn, 4 * (2 * m + cnt), kept=cnt)
    return rows


def run_c8(torch, capi, reps):
    n = 1 << 28
    src = gen.c2_uint32(torch, n)
    s, work, t = _dev(capi, torch, src, capi.U32), capi.DeviceArray(n, capi.U32), capi.Temp()
    med, mn = _time_calls(torch, lambda: capi.merge_sort_keys(work, temp=t), reps,
                          setup=lambda: work.storage.copy_(s.storage))
    out = work.storage.view(torch.int32).to(torch.int64) & 0xFFFFFFFF
    if not bool((out[1:] >= out[:-1]).all().item()) or int(out.sum().item()) != int((src.to(torch.int64) & 0xFFFFFFFF).sum().item()):
        _fail("C8 merge sort of keys")
    passes = 16  # ceil(log2(2^28 / 4096))
    rows = {"next_c8_merge_sort_u32_2p28": _row(med, mn, (1 + passes) * 8 * n, Gkeys_per_s=round(n / med / 1e6, 2),
                                                model="(1 + 16 merge passes) x 8 B/key")}
    del src, s, work, t, out
    m = 1 << 27
    keys = gen.c3_uint64(torch, m, "full")
    vals = torch.arange(m, dtype=torch.int32, device="cuda")
    sk, sv = _dev(capi, torch, keys, capi.U64), _dev(capi, torch, vals, capi.U32)
    wk, wv, t = capi.DeviceArray(m, capi.U64), capi.DeviceArray(m, capi.U32), capi.Temp()

    def setup():
        wk.storage.copy_(sk.storage)
        wv.storage.copy_(sv.storage)
    med, mn = _time_calls(torch, lambda: capi.merge_sort_pairs(wk, wv, temp=t), reps, setup=setup)
    ko, vo = wk.storage.view(torch.int64), wv.storage.view(torch.int32).to(torch.int64)
    o = ko ^ (-(1 << 63))
    if not bool((o[1:] >= o[:-1]).all().item()) or not bool((keys[vo] == ko).all().item()):
        _fail("C8 merge sort of pairs")
    passes = 15
    rows["next_c8_merge_sort_by_key_u64_u32_2p27"] = _row(med, mn, (1 + passes) * 24 * m, Gpairs_per_s=round(m / med / 1e6, 2),
                                                          model="(1 + 15 merge passes) x 24 B/pair")
    return rows


def run_all(torch, capi, reps=20):
    rows = {}
    for part in (run_c2_float, run_c3, run_c4, run_c5, run_c6, run_c7, run_c8):
        # (no empty_cache between the parts: while the driver clears gigabytes of freed memory in the
        # background, everything that is bound by bandwidth runs about 3 % slower for a few seconds)
        rows.update(part(torch, capi, reps))
    return rows
