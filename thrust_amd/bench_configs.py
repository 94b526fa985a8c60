"""The benchmark configurations beside the headline one: each is run on the device at its own
size, its result is verified there against an independent torch computation, and the whole
call (every kernel it launches, launch gaps included) is timed with events on the launch
stream.  bench.py imports this module and prints the rows inside its JSON line.

  C2  sort of 2^28 float32 keys (1 % of +-0.0 and denormals)
  C3  stable sort_by_key of 2^27 uint64 keys + uint32 values: full range / low 16 bits / 90 % one key
  C4  reduce_by_key, unique_by_key and unique over 2^28 (int32 key, float32 value), mean run 8 / 1000
  C5  copy_if and stable_partition of 2^28 float32 at 50 % / 5 % selectivity,
      merge_by_key and merge of two sorted ranges of 2^27 uint32 (+ uint32 values)

Bytes are the algorithmic ones of each call (what must be read and written once).
"""
import numpy as np

from . import datagen_device as gen

HBM_PEAK_GBS = 8000.0


def _dev(capi, torch, t, code):
    items = t.numel() * t.element_size() // np.dtype(capi.NP_DTYPES[code]).itemsize
    return capi.DeviceArray(items, code, t.view(torch.uint8))


_PAD = {}


def _time_calls(torch, fn, reps, setup=None):
    """Median and minimum device time of fn() in ms; setup() runs before each call, untimed.
    fn must not synchronise.  The device is kept busy with a fill while the host prepares
    the call, so that the first event is not reached before the call has been enqueued."""
    if "buf" not in _PAD:
        _PAD["buf"] = torch.empty(1 << 30, dtype=torch.uint8, device="cuda")
    if setup:
        setup()
    fn()  # sizes temp storage, warms up
    torch.cuda.synchronize()
    times = []
    for _ in range(reps):
        if setup:
            setup()
        _PAD["buf"].zero_()
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
        rows[f"c3_sort_by_key_u64_u32_2p27_{kind}"] = _row(
            med, mn, 200 * m, Gpairs_per_s=round(m / med / 1e6, 2),
            model="200 B/pair: histogram read + 8 passes x 24 B; passes over a constant digit are skipped")
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
        rows[f"c5_stable_partition_{tag}"] = _row(med, mn, 8 * n, selected=cnt)
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


def run_all(torch, capi, reps=5):
    rows = {}
    for part in (run_c2_float, run_c3, run_c4, run_c5):
        rows.update(part(torch, capi, reps))
        torch.cuda.empty_cache()
    _PAD.clear()
    torch.cuda.empty_cache()
    return rows
