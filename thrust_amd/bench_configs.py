#!/usr/bin/env python3
"""Timings of the benchmark configurations beside the headline one, on one GPU.

For each configuration the device-side time of one call is reported as the sum of the
library's own per-kernel event timers (inputs resident in HBM, temp storage sized once),
with the algorithmic bytes of the call and the resulting fraction of the 8 TB/s HBM peak:

  C2  sort of 2^28 float32 keys
  C3  sort_by_key of 2^27 uint64 keys + uint32 values: full range / low 16 bits / 90 % one key
  C4  reduce_by_key and unique_by_key over 2^28 (int32 key, float32 value), mean run 8 / 1000
  C5  copy_if and stable_partition of 2^28 float32 at 50 % / 5 % selectivity,
      merge and merge_by_key of two sorted ranges of 2^27 uint32 (+ uint32 values)
  C6  callers on either side of the path: count_if, inner_product, transform_reduce and
      the transform scans over 2^28 int32 / float32, inclusive and exclusive scan_by_key
      over 2^28 (int32 key, float32 value)

  C7  the four set operations on two sorted ranges of 2^27 uint32 with runs of about four
      and two equal keys (bytes: both inputs read, the result written)
  C8  the stable comparison sort (merge sort) of 2^28 uint32 keys and of 2^27 uint64 keys
      with uint32 values (bytes: one block sort and ceil(log2(n / 4096)) merge passes, each
      reading and writing every element)

Inputs are generated on the device from a seeded generator.  Usage:
  python3 thrust_amd/bench_configs.py [c2] [c3] [c4] [c5] [c6] [c7] [c8]
"""
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

HBM_PEAK_GBS = 8000.0
REPS = 5


def main():
    import torch
    from thrust_amd import capi
    if not torch.cuda.is_available():
        raise SystemExit("bench_configs.py needs a GPU")
    capi.load()
    which = [a.lower() for a in sys.argv[1:]] or ["c2", "c3", "c4", "c5", "c6", "c7", "c8"]
    g = torch.Generator(device="cuda")
    g.manual_seed(1)

    def dev(t, code):
        items = t.numel() * t.element_size() // np.dtype(capi.NP_DTYPES[code]).itemsize
        return capi.DeviceArray(items, code, t.view(torch.uint8))

    def run(name, fn, nbytes, setup=None, extra=""):
        if setup:
            setup()
        fn()  # sizes temp storage, warms up
        torch.cuda.synchronize()
        capi.profile_enable(True)
        for _ in range(REPS):
            if setup:
                setup()
            fn()
        torch.cuda.synchronize()
        prof = capi.profile_collect()
        capi.profile_enable(False)
        ms = sum(v[1] for v in prof.values()) / REPS
        kernels = "  ".join(f"{k}={v[1] / REPS:.3f}" for k, v in prof.items())
        gbs = nbytes / ms / 1e6
        print(f"{name:44s} {ms:8.3f} ms {gbs:8.0f} GB/s {gbs / HBM_PEAK_GBS * 100:5.1f}%  {extra}  [{kernels}]",
              flush=True)

    n = 1 << 28
    if "c2" in which:
        f = (torch.rand(n, device="cuda", generator=g) * 2e6 - 1e6).float()
        src, work, t = dev(f, capi.F32), capi.DeviceArray(n, capi.F32), capi.Temp()
        run("C2 sort f32 2^28", lambda: capi.sort_keys(work, temp=t), 36 * n,
            setup=lambda: work.storage.copy_(src.storage), extra="36 B/key")
        del f, src, work, t
    if "c3" in which:
        m = 1 << 27
        for kind in ("full", "low16", "skew90"):
            r = torch.randint(-(1 << 62), 1 << 62, (m,), dtype=torch.int64, device="cuda", generator=g) * 2 \
                + torch.randint(0, 2, (m,), dtype=torch.int64, device="cuda", generator=g)
            if kind == "low16":
                r = r & 0xFFFF
            if kind == "skew90":
                pick = torch.randint(0, 10, (m,), device="cuda", generator=g)
                r = torch.where(pick != 0, torch.full_like(r, 0x0123456789ABCDEF), r)
            v = torch.arange(m, dtype=torch.int32, device="cuda")
            sk, sv = dev(r, capi.U64), dev(v, capi.U32)
            wk, wv, t = capi.DeviceArray(m, capi.U64), capi.DeviceArray(m, capi.U32), capi.Temp()

            def setup():
                wk.storage.copy_(sk.storage)
                wv.storage.copy_(sv.storage)
            # model: histogram read + 8 passes reading and writing 12 B per pair
            run(f"C3 sort_by_key u64+u32 2^27 {kind}", lambda: capi.sort_pairs(wk, wv, temp=t), 200 * m,
                setup=setup, extra="200 B/pair when all 8 passes run")
            del r, v, sk, sv, wk, wv, t
    if "c4" in which:
        for mean in (8, 1000):
            nseg = int(n / mean * 1.2) + 1000
            u = torch.rand(nseg, device="cuda", generator=g, dtype=torch.float64).clamp_(1e-12, 1.0)
            lens = (torch.floor(torch.log(u) / np.log1p(-1.0 / mean)) + 1).long()
            keys = torch.repeat_interleave(torch.arange(nseg, device="cuda", dtype=torch.int32), lens)[:n].contiguous()
            if keys.numel() != n:
                raise SystemExit("bench_configs: segment generator came up short")
            runs = int(keys[-1].item()) + 1
            vals = torch.rand(n, device="cuda", generator=g)
            dk, dv = dev(keys, capi.I32), dev(vals, capi.F32)
            ko, vo, t = capi.DeviceArray(n, capi.I32), capi.DeviceArray(n, capi.F32), capi.Temp()
            run(f"C4 reduce_by_key mean run {mean}",
                lambda: capi.reduce_by_key(dk, dv, temp=t, keys_out=ko, values_out=vo), 8 * n + 8 * runs)
            run(f"C4 unique_by_key mean run {mean}",
                lambda: capi.unique_by_key(dk, dv, keys_out=ko, values_out=vo, temp=t), 8 * n + 8 * runs)
            run(f"C4 unique (keys only) mean run {mean}",
                lambda: capi.unique(dk, out=ko, temp=t), 4 * n + 4 * runs)
            del keys, vals, dk, dv, ko, vo, t, u, lens
    if "c5" in which:
        x = torch.rand(n, device="cuda", generator=g)
        dx, out, work = dev(x, capi.F32), capi.DeviceArray(n, capi.F32), capi.DeviceArray(n, capi.F32)
        t, tp = capi.Temp(), capi.Temp()
        for thr in (0.5, 0.05):
            _, cnt = capi.copy_if(dx, capi.LT, thr, out=out, temp=t)
            run(f"C5 copy_if x<{thr}", lambda: capi.copy_if(dx, capi.LT, thr, out=out, temp=t), 4 * n + 4 * cnt)
            run(f"C5 stable_partition x<{thr}", lambda: capi.stable_partition(work, capi.LT, thr, temp=tp), 8 * n,
                setup=lambda: work.storage.copy_(dx.storage))
        del x, dx, out, work, t, tp
        m = 1 << 27

        def sorted_u32():
            r = torch.randint(-(1 << 31), 1 << 31, (m,), dtype=torch.int32, device="cuda", generator=g)
            return torch.sort(r.to(torch.int64) & 0xFFFFFFFF)[0].to(torch.int32)
        ka, kb = sorted_u32(), sorted_u32()
        va = torch.arange(m, dtype=torch.int32, device="cuda")
        vb = va + m
        a = [dev(z, capi.U32) for z in (ka, kb, va, vb)]
        ko, vo, t, t2 = capi.DeviceArray(2 * m, capi.U32), capi.DeviceArray(2 * m, capi.U32), capi.Temp(), capi.Temp()
        run("C5 merge_by_key 2 x 2^27 u32+u32",
            lambda: capi.merge_by_key(*a, temp=t, keys_out=ko, values_out=vo), 16 * 2 * m)
        run("C5 merge 2 x 2^27 u32", lambda: capi.merge(a[0], a[1], out=ko, temp=t2), 8 * 2 * m)
        del ka, kb, va, vb, a, ko, vo, t, t2
    if "c6" in which:
        x = torch.randint(0, 1001, (n,), dtype=torch.int32, device="cuda", generator=g)
        dx, t = dev(x, capi.I32), capi.Temp()
        run("C6 count_if i32 x<500", lambda: capi.count_if(dx, capi.LT, 500, temp=t), 4 * n)
        f1 = torch.rand(n, device="cuda", generator=g)
        f2 = torch.rand(n, device="cuda", generator=g)
        d1, d2, t2, out1 = dev(f1, capi.F32), dev(f2, capi.F32), capi.Temp(), capi.DeviceArray(1, capi.F32)
        run("C6 inner_product f32", lambda: capi.inner_product(d1, d2, init=0.0, temp=t2, out=out1), 8 * n)
        t3, t4, so, so_i = capi.Temp(), capi.Temp(), capi.DeviceArray(n, capi.F32), capi.DeviceArray(n, capi.I32)
        run("C6 transform_reduce f32 square, plus",
            lambda: capi.transform_reduce(d1, capi.SQUARE, init=0.0, temp=t3, out=out1), 4 * n)
        run("C6 transform_inclusive_scan f32 negate, plus",
            lambda: capi.transform_inclusive_scan(d1, capi.NEGATE, out=so, temp=t4), 8 * n)
        run("C6 transform_exclusive_scan i32 square, plus",
            lambda: capi.transform_exclusive_scan(dx, capi.SQUARE, init=3, out=so_i, temp=t4), 8 * n)
        del x, dx, f1, f2, d1, d2, t, t2, t3, t4, so, so_i
        mean = 8
        nseg = int(n / mean * 1.2) + 1000
        u = torch.rand(nseg, device="cuda", generator=g, dtype=torch.float64).clamp_(1e-12, 1.0)
        lens = (torch.floor(torch.log(u) / np.log1p(-1.0 / mean)) + 1).long()
        keys = torch.repeat_interleave(torch.arange(nseg, device="cuda", dtype=torch.int32), lens)[:n].contiguous()
        vals = torch.rand(n, device="cuda", generator=g)
        dk, dv, vo, t = dev(keys, capi.I32), dev(vals, capi.F32), capi.DeviceArray(n, capi.F32), capi.Temp()
        run("C6 inclusive_scan_by_key mean run 8", lambda: capi.inclusive_scan_by_key(dk, dv, out=vo, temp=t), 12 * n)
        run("C6 exclusive_scan_by_key mean run 8",
            lambda: capi.exclusive_scan_by_key(dk, dv, init=0.0, out=vo, temp=t), 12 * n)
    if "c7" in which:
        m = 1 << 27

        def sorted_keys(distinct):
            r = torch.randint(0, distinct, (m,), dtype=torch.int32, device="cuda", generator=g)
            return torch.sort(r)[0]
        ka, kb = sorted_keys(m // 4), sorted_keys(m // 2)
        da, db = dev(ka, capi.U32), dev(kb, capi.U32)
        out, t = capi.DeviceArray(2 * m, capi.U32), capi.Temp()
        names = ("set_difference", "set_intersection", "set_symmetric_difference", "set_union")
        for op, name in enumerate(names):
            _, cnt = capi.set_operation(op, da, db, out=out, temp=t)
            run(f"C7 {name} 2 x 2^27 u32", lambda: capi.set_operation(op, da, db, out=out, temp=t),
                4 * (2 * m + cnt), extra=f"{cnt} out")
        va = torch.arange(m, dtype=torch.int32, device="cuda")
        dva, dvb, vo, t2 = dev(va, capi.U32), dev(va + m, capi.U32), capi.DeviceArray(2 * m, capi.U32), capi.Temp()
        _, _, cnt = capi.set_operation_by_key(3, da, db, dva, dvb, keys_out=out, values_out=vo, temp=t2)
        run("C7 set_union_by_key 2 x 2^27 u32+u32",
            lambda: capi.set_operation_by_key(3, da, db, dva, dvb, keys_out=out, values_out=vo, temp=t2),
            4 * (2 * m + cnt) + 8 * cnt, extra=f"{cnt} out")
        del ka, kb, da, db, out, t, va, dva, dvb, vo, t2
    if "c8" in which:
        def passes(count):
            return 1 + int(np.ceil(np.log2(max(1.0, count / 4096))))
        r = torch.randint(-(1 << 31), 1 << 31, (n,), dtype=torch.int32, device="cuda", generator=g)
        src, work, t = dev(r, capi.U32), capi.DeviceArray(n, capi.U32), capi.Temp()
        run("C8 comparison sort u32 2^28", lambda: capi.merge_sort_keys(work, temp=t), passes(n) * 8 * n,
            setup=lambda: work.storage.copy_(src.storage), extra=f"{passes(n)} x 8 B/key")
        del r, src, work, t
        m = 1 << 27
        r = torch.randint(-(1 << 62), 1 << 62, (m,), dtype=torch.int64, device="cuda", generator=g)
        v = torch.arange(m, dtype=torch.int32, device="cuda")
        sk, sv = dev(r, capi.U64), dev(v, capi.U32)
        wk, wv, t = capi.DeviceArray(m, capi.U64), capi.DeviceArray(m, capi.U32), capi.Temp()

        def setup():
            wk.storage.copy_(sk.storage)
            wv.storage.copy_(sv.storage)
        run("C8 comparison sort_by_key u64+u32 2^27", lambda: capi.merge_sort_pairs(wk, wv, temp=t),
            passes(m) * 24 * m, setup=setup, extra=f"{passes(m)} x 24 B/pair")


if __name__ == "__main__":
    main()
