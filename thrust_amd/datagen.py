"""Seeded synthetic inputs for the benchmark configurations.

Counter-based: element i of a stream is a pure function of (seed, i) -- SplitMix64 applied
to seed * 2^32 + i -- so the same bytes can be produced in chunks, on any machine, in
numpy.  (std::uniform_*_distribution is library-specific and therefore not used.)
"""
import numpy as np

_M64 = (1 << 64) - 1


def splitmix64(seed, n, start=0):
    """uint64[n]: SplitMix64 finaliser of the counters (seed<<32) + start + i."""
    with np.errstate(over="ignore"):
        z = np.arange(start, start + n, dtype=np.uint64)
        z += np.uint64((seed << 32) & _M64)
        z += np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        z ^= z >> np.uint64(31)
    return z


def _chunks(n, chunk=1 << 24):
    for s in range(0, n, chunk):
        yield s, min(chunk, n - s)


def _build(n, dtype, fn):
    out = np.empty(n, dtype)
    for s, c in _chunks(n):
        out[s:s + c] = fn(s, c)
    return out


def u01(seed, n, start=0):
    """float32 uniform in [0, 1): top 24 bits of the stream."""
    return ((splitmix64(seed, n, start) >> np.uint64(40)).astype(np.float32)
            * np.float32(1.0 / (1 << 24)))


def c1_int32(n, seed=42):
    """Config 1: int32 uniform in [0, 1000]."""
    return _build(n, np.int32, lambda s, c: (splitmix64(seed, c, s) % np.uint64(1001)).astype(np.int32))


def c2_uint32(n, seed=1):
    """Config 2a: uint32 over the full range."""
    return _build(n, np.uint32, lambda s, c: (splitmix64(seed, c, s) >> np.uint64(32)).astype(np.uint32))


def c2_float32(n, seed=2):
    """Config 2b: float32 uniform in [-1e6, 1e6] with 1% of +0.0 / -0.0 / +-denormals."""
    def gen(s, c):
        f = (np.float32(-1e6) + np.float32(2e6) * u01(seed, c, s)).astype(np.float32)
        r = splitmix64(seed + 1000, c, s)
        special = (r % np.uint64(100)) == 0
        kind = (r >> np.uint64(8)) % np.uint64(4)
        sign = ((r >> np.uint64(16)) & np.uint64(1)).astype(np.uint32) << np.uint32(31)
        mant = ((r >> np.uint64(20)) % np.uint64(0x7FFFFF) + np.uint64(1)).astype(np.uint32)
        bits = np.where(kind == 0, np.uint32(0),
                        np.where(kind == 1, np.uint32(0x80000000), mant | sign)).astype(np.uint32)
        fb = f.view(np.uint32).copy()
        fb[special] = bits[special]
        return fb.view(np.float32)
    return _build(n, np.float32, gen)


C3_CONSTANT = 0x0123456789ABCDEF


def c3_uint64(n, kind, seed=3):
    """Config 3 keys: kind in {"full", "low16", "skew90"}."""
    def gen(s, c):
        r = splitmix64(seed, c, s)
        if kind == "full":
            return r
        if kind == "low16":
            return r & np.uint64(0xFFFF)
        if kind == "skew90":
            pick = splitmix64(seed + 1000, c, s) % np.uint64(10)
            return np.where(pick != 0, np.uint64(C3_CONSTANT), r)
        raise ValueError(kind)
    return _build(n, np.uint64, gen)


def c4_segments(n, mean, seed=4):
    """Config 4: (int32 keys, float32 values); keys = run index, run lengths ~ Geometric(1/mean)."""
    p = 1.0 / mean
    keys = np.empty(n, np.int32)
    filled, run, start = 0, 0, 0
    log1mp = np.log1p(-p)
    while filled < n:
        c = 1 << 20
        u = (splitmix64(seed, c, start).astype(np.float64) + 0.5) / float(1 << 64)
        start += c
        lens = np.floor(np.log(u) / log1mp).astype(np.int64) + 1
        ends = np.cumsum(lens)
        take = min(int(np.searchsorted(ends, n - filled, side="left")) + 1, c)
        lens = lens[:take]
        ids = np.repeat(np.arange(run, run + take, dtype=np.int64), lens)[: n - filled]
        keys[filled:filled + ids.size] = ids.astype(np.int32)
        filled += ids.size
        run += take
    vals = _build(n, np.float32, lambda s, c: u01(seed + 1000, c, s))
    return keys, vals


def c5_float32(n, seed=5):
    """Config 5: float32 uniform in [0, 1)."""
    return _build(n, np.float32, lambda s, c: u01(seed, c, s))


def c5_merge_inputs(n_each, seed=6):
    """Config 5 merge: two sorted uint32 arrays and their payloads (original index)."""
    out = []
    for j in range(2):
        k = c2_uint32(n_each, seed + j)
        order = np.argsort(k, kind="stable").astype(np.uint32)
        out.append((k[order], order))
    return out
