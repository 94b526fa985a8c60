#!/usr/bin/env python3
"""Headline benchmark: the sort of 2^28 uint32 keys (the configuration the headline metric is quoted on) on one MI355X,
through thrust_amd_sort_keys, the C-ABI entry point that thrust::sort calls for arithmetic keys, with
thrust_amd_reduce / thrust_amd_inclusive_scan over 2^28 int32 measured beside it.

One step = one full radix sort of a device-resident, never-before-sorted copy of the seeded
input (the sort is in place, so every step gets its own copy; the copies are made before the
timed region).  Exactly K steps are timed between two device synchronisations; the printed
JSON line follows the driver's contract.  `roofline` describes the dominant kernel (one
onesweep digit-binning pass: n keys read + n keys written), timed with events on the launch
stream; `cpu_baseline` is the reference's own OpenMP device system (oracle/_ref, built from
the reference sources) when that library travelled with the tree, else the C restatement,
timed on this machine's host cores on the very keys and values the GPU legs used.  `configs`
holds one verified row per other benchmark configuration (thrust_amd/bench_configs.py).
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published
N_SORT = 1 << 28
N_C1 = 1 << 28

# HBM bytes per onesweep pass launch at n = 2^28 uint32 come from the committed counter summary:
# rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this very command, each scaled by what the same counter
# reads for kernels of known size in the same run (FETCH_SIZE reports half the KiB fetched: x2.0 from
# the reduce kernel's 1 GiB; WRITE_SIZE x1.0 from the scan kernel's 1 GiB).
PMC_SUMMARY = os.path.join("profiles", "bench_kernels_pmc_counters.txt")
FETCH_SCALE, WRITE_SCALE = 2.0, 1.0


def pass_traffic_from_profile():
    """(bytes per launch, "file:line") of the uint32 keys-only onesweep pass in the committed counter
    summary, or (None, reason) when the file or the line is not there."""
    import re
    path = os.path.join(ROOT, PMC_SUMMARY)
    try:
        lines = open(path).read().splitlines()
    except OSError:
        return None, f"{PMC_SUMMARY} not found"
    for i, text in enumerate(lines):
        if text.startswith("onesweep_pass_kernel<unsigned int, unsigned int, false"):
            for j in range(i + 1, min(i + 4, len(lines))):
                m = re.search(r"FETCH (\d+) KiB WRITE (\d+) KiB", lines[j])
                if m:
                    nbytes = (FETCH_SCALE * int(m.group(1)) + WRITE_SCALE * int(m.group(2))) * 1024.0
                    return nbytes, f"{PMC_SUMMARY}:{j + 1}"
    return None, f"no onesweep_pass line in {PMC_SUMMARY}"


def device_random_u32(torch, n, seed):
    """uint32 keys, uniform over the full range: the seeded counter-based stream of
    thrust_amd.datagen.c2_uint32, produced on the device (same bytes)."""
    from thrust_amd import datagen_device
    return datagen_device.c2_uint32(torch, n, seed).view(torch.uint8)


def time_region(torch, fn, steps, warmup):
    for i in range(warmup):
        fn(i, True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        fn(i, False)
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / steps


def bench_sort(torch, capi, steps, warmup, want_host_copy):
    n = N_SORT
    src = device_random_u32(torch, n, 1)
    temp = capi.Temp()
    bufs = [capi.DeviceArray(n, capi.U32, src.clone()) for _ in range(steps)]
    warm = [capi.DeviceArray(n, capi.U32, src.clone()) for _ in range(max(warmup, 1))]
    capi.sort_keys(warm[0], temp=temp)  # sizes the temp storage once

    def step(i, is_warm):
        capi.sort_keys(warm[i] if is_warm else bufs[i], temp=temp)

    ms = time_region(torch, step, steps, warmup)
    # parity spot-check of the last sorted buffer: order + multiset (checksum) preserved
    out = bufs[-1].storage.view(torch.int32).to(torch.int64) & 0xFFFFFFFF
    inp = src.view(torch.int32).to(torch.int64) & 0xFFFFFFFF
    ok = bool((out[1:] >= out[:-1]).all().item()) and int(out.sum().item()) == int(inp.sum().item())
    if not ok:
        raise SystemExit("bench: sorted output failed the order/checksum check")
    del bufs, warm
    host_keys = src.cpu().numpy().view(np.uint32) if want_host_copy else None

    # per-kernel durations of the same call, events on the launch stream.  Three unprofiled sorts of
    # fresh copies run first: right behind the burst of copies that makes the inputs the first
    # launches read up to 15 % longer than in the timed loop.
    reps = 5
    prof_bufs = [capi.DeviceArray(n, capi.U32, src.clone()) for _ in range(reps)]
    settle = [capi.DeviceArray(n, capi.U32, src.clone()) for _ in range(3)]
    torch.cuda.synchronize()
    for b in settle:
        capi.sort_keys(b, temp=temp)
    torch.cuda.synchronize()
    del settle
    capi.profile_enable(True)
    for b in prof_bufs:
        capi.sort_keys(b, temp=temp)
    torch.cuda.synchronize()
    prof = capi.profile_collect()
    capi.profile_enable(False)
    launches, total_ms = prof["onesweep_pass"]
    pass_ms = total_ms / launches
    kernels_ms = {k: v[1] / reps for k, v in prof.items()}
    return ms, pass_ms, kernels_ms, host_keys


class C1:
    """reduce and inclusive_scan over 2^28 int32: buffers made once and measured twice -- before and
    after the sort -- so that a disturbance at either end of the run does not decide the figure;
    the mean of the two passes is the figure reported, the better pass and both passes are printed."""

    def __init__(self, torch, capi, want_host_copy):
        from thrust_amd import datagen_device
        self.torch, self.capi, n = torch, capi, N_C1
        x = datagen_device.c1_int32(torch, n)  # the stream of thrust_amd.datagen.c1_int32 (seed 42)
        self.d = capi.DeviceArray(n, capi.I32, x.view(torch.uint8))
        self.out1 = capi.DeviceArray(1, capi.I32)
        self.outn = capi.DeviceArray(n, capi.I32)
        self.t_r, self.t_s = capi.Temp(), capi.Temp()
        capi.reduce(self.d, temp=self.t_r, out=self.out1)
        capi.inclusive_scan(self.d, out=self.outn, temp=self.t_s)
        total = int(x.sum(dtype=torch.int64).item())
        got = int(self.out1.numpy()[0])
        if (got - total) % (1 << 32) != 0:
            raise SystemExit("bench: reduce result differs from the int64 sum modulo 2^32")
        last = int(self.outn.storage.view(torch.int32)[n - 1].item())
        if (last - total) % (1 << 32) != 0:
            raise SystemExit("bench: inclusive_scan total differs from the int64 sum modulo 2^32")
        self.host = x.cpu().numpy() if want_host_copy else None
        self.passes = []
        self.copy_ms = []
        self.static_ms = []

    def measure(self, steps, warmup):
        # calls of 0.2 - 0.4 ms: at least 50 back to back, so that the one synchronisation at the end
        # of the timed region does not weigh on the figure
        reps = max(steps, 50)
        # and at least 20 untimed calls first: three calls of 0.2 ms end before the device has left its
        # idle clocks
        warmup = max(warmup, 20)
        capi = self.capi
        ms_reduce = time_region(self.torch, lambda i, w: capi.reduce(self.d, temp=self.t_r, out=self.out1), reps, warmup)
        ms_scan = time_region(self.torch, lambda i, w: capi.inclusive_scan(self.d, out=self.outn, temp=self.t_s), reps, warmup)
        # a plain device copy of the same 1 GiB into the same output (torch's copy kernel): what moving the
        # scan's bytes costs with no scan in between
        src_t, dst_t = self.d.storage, self.outn.storage
        self.copy_ms.append(time_region(self.torch, lambda i, w: dst_t.copy_(src_t), reps, warmup))
        # the same scan through the entry point that keeps its tile descriptors in the library's own
        # storage and therefore needs no clearing launch in front of the kernel
        self.static_ms.append(time_region(self.torch, lambda i, w: capi.inclusive_scan_static(self.d, out=self.outn), reps, warmup))
        self.passes.append((ms_reduce, ms_scan))

    def mean(self):
        return sum(p[0] for p in self.passes) / len(self.passes), sum(p[1] for p in self.passes) / len(self.passes)

    def best(self):
        return min(p[0] for p in self.passes), min(p[1] for p in self.passes)


def _timed(fn, warmups, reps):
    for _ in range(warmups):
        fn()
    ts = []
    for _ in range(reps):
        t0 = time.perf_counter()
        fn()
        ts.append(time.perf_counter() - t0)
    ts.sort()
    return ts[0], ts[len(ts) // 2]


def cpu_baseline(sort_keys, c1_values):
    """The reference's OpenMP device system (or the restatement) on the host cores, on the
    configuration itself: the very keys and values the GPU legs used (downloaded from the
    device), 2^28 elements each; 1 warm-up + 2 timed sorts, 1 warm-up + 5 timed reduces and
    scans; minimum and median.  The other rows' figures are on 2^24-element samples."""
    from oracle import cpu as ocpu
    from thrust_amd import datagen
    cores = len(os.sched_getaffinity(0))
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    if ocpu.ref_available("omp"):
        impl, kind = ocpu.Reference("omp"), "reference"
    else:
        if not os.path.exists(ocpu.ORACLE_LIB):
            ocpu.build(with_ref=False)
        impl, kind = ocpu.Oracle(), "port"
    n = sort_keys.size
    out = {}
    t_min, t_med = _timed(lambda: out.update(s=impl.sort_keys(sort_keys)), 1, 2)
    if not np.all(out["s"][:-1] <= out["s"][1:]):
        raise SystemExit("bench: CPU baseline output is not sorted")
    del out
    r_min, r_med = _timed(lambda: impl.reduce(c1_values), 1, 5)
    s_min, s_med = _timed(lambda: impl.inclusive_scan(c1_values), 1, 5)
    # the other rows of the path on 2^24-element samples of their configurations (GB/s of the
    # same algorithmic bytes the GPU figures use; 1 warm-up + 2 timed calls, minimum)
    m = 1 << 24

    def gbs(nbytes, fn):
        return round(nbytes / _timed(fn, 1, 2)[0] / 1e9, 3)
    ck, cv = datagen.c4_segments(m, 8)
    runs = int(ck[-1]) + 1
    f = datagen.c5_float32(m)
    (ka, va), (kb, vb) = datagen.c5_merge_inputs(m // 2)
    rows = {
        "reduce_by_key_GBps": gbs(8.0 * m + 8.0 * runs, lambda: impl.reduce_by_key(ck, cv)),
        "unique_by_key_GBps": gbs(8.0 * m + 8.0 * runs, lambda: impl.unique_by_key(ck, cv)),
        "copy_if_half_GBps": gbs(6.0 * m, lambda: impl.copy_if(f, ocpu.LT, 0.5)),
        "stable_partition_half_GBps": gbs(8.0 * m, lambda: impl.stable_partition(f.copy(), ocpu.LT, 0.5)),
        "merge_by_key_GBps": gbs(16.0 * m, lambda: impl.merge_by_key(ka, kb, va, vb)),
    }
    return {
        "value": round(n / t_med / 1e9, 4), "unit": "Gkeys/s", "cores": cores, "kind": kind,
        "sample": f"thrust::sort of the same 2^{n.bit_length() - 1} uint32 keys the GPU sorted (the whole "
                  "configuration), 1 warm-up + 2 timed calls, median; each call includes one copy of the "
                  "input made by the binding",
        "sort_s": {"min": round(t_min, 3), "median": round(t_med, 3)},
        "reduce_i32_2p28": {"GBps": round(4.0 * c1_values.size / r_med / 1e9, 2),
                            "ms_min": round(r_min * 1e3, 2), "ms_median": round(r_med * 1e3, 2)},
        "inclusive_scan_i32_2p28": {"GBps": round(8.0 * c1_values.size / s_med / 1e9, 2),
                                    "ms_min": round(s_min * 1e3, 2), "ms_median": round(s_med * 1e3, 2)},
        "rows_2p24": rows,
        "note": "OMP back end: sort = per-thread LSD radix + serial pairwise merges; "
                "inclusive_scan is single-threaded by construction",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-configs", action="store_true",
                    help="skip the verified rows of the other configurations (C2 float, C3, C4, C5)")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py: this build measures one GPU only (the device system is "
                         "single-GPU by design); run with --gpus 1")
    if not 1 <= args.steps <= 200:
        raise SystemExit("bench.py: --steps must be in [1, 200] (each step sorts its own 1 GiB copy)")

    import torch
    from thrust_amd import capi
    if not torch.cuda.is_available():
        raise SystemExit("bench.py needs a GPU")
    capi.load()  # raises if the HIP library is missing: there is no fallback

    want_host = not args.no_cpu_baseline
    # Nothing in this run gives device memory back to the driver (no empty_cache): for a few seconds after
    # gigabytes have been freed, a pure read runs 3 % slower (0.183 against 0.176 ms for the same reduce on
    # the same buffer, back to 0.176 ms three seconds later -- measured), presumably while the freed memory
    # is cleared in the background.  torch's caching allocator hands the blocks from one part to the next.
    c1 = C1(torch, capi, want_host)
    c1.measure(args.steps, args.warmup)
    ms_sort, pass_ms, kernels_ms, host_keys = bench_sort(torch, capi, args.steps, args.warmup, want_host)
    c1.measure(args.steps, args.warmup)
    ms_reduce, ms_scan = c1.mean()
    best_reduce, best_scan = c1.best()
    ms_copy = sum(c1.copy_ms) / len(c1.copy_ms)
    ms_static = sum(c1.static_ms) / len(c1.static_ms)
    host_c1 = c1.host
    c1_passes = [{"reduce_ms": round(r, 4), "scan_ms": round(sc, 4)} for r, sc in c1.passes]
    del c1
    config_rows = None
    if not args.no_configs:
        from thrust_amd import bench_configs
        config_rows = bench_configs.run_all(torch, capi)

    n = N_SORT
    gkeys = n / ms_sort / 1e6
    pass_bytes = 2.0 * 4.0 * n  # keys read + keys written by one digit-binning pass
    pass_gbs = pass_bytes / pass_ms / 1e6
    traffic, traffic_source = pass_traffic_from_profile()
    line = {
        "metric": "sort Gkeys/s (2^28 u32) + scan/reduce GB/s as % of HBM peak, 1 GPU",
        "value": round(gkeys, 3),
        "unit": "Gkeys/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_sort, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u32",
        "data": "synthetic",
        "config": {"workload": "thrust_amd_sort_keys (the C-ABI entry point behind thrust::sort), N=2^28 uint32 keys "
                               "uniform over the full range (seeded), in place, keys resident in HBM"},
        "sort_model_bytes_pct_of_peak": round(36.0 * n / ms_sort / 1e6 / HBM_PEAK_GBS * 100, 2),
        "sort_kernels_ms": {k: round(v, 4) for k, v in kernels_ms.items()},
        "sort_kernels_ms_note": "each launch of a separate profiled run bracketed by its own pair of events: the pairs "
                                "add about 4 % per launch, so these sum to more than ms_per_step, which has none",
        "reduce_i32_2p28": {"ms": round(ms_reduce, 4), "GBps": round(4.0 * N_C1 / ms_reduce / 1e6, 1),
                            "pct_of_peak": round(4.0 * N_C1 / ms_reduce / 1e6 / HBM_PEAK_GBS * 100, 2),
                            "ms_best": round(best_reduce, 4),
                            "pct_of_peak_best": round(4.0 * N_C1 / best_reduce / 1e6 / HBM_PEAK_GBS * 100, 2)},
        "inclusive_scan_i32_2p28": {"ms": round(ms_scan, 4), "GBps": round(8.0 * N_C1 / ms_scan / 1e6, 1),
                                    "pct_of_peak": round(8.0 * N_C1 / ms_scan / 1e6 / HBM_PEAK_GBS * 100, 2),
                                    "ms_best": round(best_scan, 4),
                                    "pct_of_peak_best": round(8.0 * N_C1 / best_scan / 1e6 / HBM_PEAK_GBS * 100, 2),
                                    # beside it: a plain copy of the same bytes in this run, and the best hand-written
                                    # copy kernel of profiles/copy_ceiling.txt (256 threads x 16 bytes: 0.3459 ms)
                                    "torch_copy_ms": round(ms_copy, 4),
                                    "pct_of_torch_copy": round(ms_copy / ms_scan * 100, 1),
                                    "pct_of_best_copy_kernel": round(0.3459 / ms_scan * 100, 1)},
        "inclusive_scan_static_i32_2p28": {"ms": round(ms_static, 4), "GBps": round(8.0 * N_C1 / ms_static / 1e6, 1),
                                           "pct_of_peak": round(8.0 * N_C1 / ms_static / 1e6 / HBM_PEAK_GBS * 100, 2),
                                           "note": "thrust_amd_inclusive_scan_static: descriptors in the library's own "
                                                   "storage, kept clean by the kernel itself, one launch per call"},
        # before and after the sort, each the mean of >= 50 back-to-back calls; "ms" above is the mean of the two
        "reduce_scan_passes": c1_passes,
        "roofline": {"bound": "hbm", "kernel": "onesweep_pass (one of 4 per sort)",
                     "achieved": round(pass_gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(pass_gbs / HBM_PEAK_GBS, 4), "traffic": traffic, "traffic_source": traffic_source,
                     "launch_ms": round(pass_ms, 4)},
    }
    if config_rows is not None:
        line["configs"] = config_rows
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(host_keys, host_c1)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
