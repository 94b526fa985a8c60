"""The seeded benchmark inputs of datagen.py, produced with torch on the device.

Same counter-based streams (SplitMix64 of seed * 2^32 + i), computed in two's-complement
int64 arithmetic, so uint32 / uint64 / int32 / float32 streams hold the same bytes as the
numpy versions (tests/test_oracle.py compares them on the CPU).  The config-4 run lengths
go through log() in float64 and may differ from numpy's in the last place of a quotient;
they follow the same distribution and are not meant to be compared byte for byte.
Unsigned values travel as the int32 / int64 tensors with the same bits.
"""
import numpy as np

from . import datagen

_C0 = 0x9E3779B97F4A7C15
_C1 = 0xBF58476D1CE4E5B9
_C2 = 0x94D049BB133111EB


def _s64(x):
    """Python int -> the int64 with the same low 64 bits."""
    x &= (1 << 64) - 1
    return x - (1 << 64) if x >= (1 << 63) else x


def _lsr(torch, z, k):
    """Logical shift right of the 64-bit patterns in an int64 tensor."""
    return (z >> k) & ((1 << (64 - k)) - 1)


def splitmix64(torch, seed, n, start=0, device="cuda"):
    """int64[n] holding the uint64 stream of datagen.splitmix64(seed, n, start)."""
    z = torch.arange(start, start + n, dtype=torch.int64, device=device)
    z += _s64((seed << 32) + _C0)
    z = (z ^ _lsr(torch, z, 30)) * _s64(_C1)
    z = (z ^ _lsr(torch, z, 27)) * _s64(_C2)
    z ^= _lsr(torch, z, 31)
    return z


def _umod(torch, z, m):
    """(uint64 pattern of z) mod m, for small m, as non-negative int64."""
    return ((_lsr(torch, z, 1) % m) * 2 + (z & 1)) % m


def _chunked(torch, n, dtype, fn, device, chunk=1 << 26):
    out = torch.empty(n, dtype=dtype, device=device)
    for s in range(0, n, chunk):
        c = min(chunk, n - s)
        out[s:s + c] = fn(s, c)
    return out


def u01(torch, seed, n, start=0, device="cuda"):
    return _lsr(torch, splitmix64(torch, seed, n, start, device), 40).to(torch.float32) * float(1.0 / (1 << 24))


def c1_int32(torch, n, seed=42, device="cuda"):
    return _chunked(torch, n, torch.int32,
                    lambda s, c: _umod(torch, splitmix64(torch, seed, c, s, device), 1001).to(torch.int32), device)


def c2_uint32(torch, n, seed=1, device="cuda"):
    """int32 tensor with the bits of datagen.c2_uint32."""
    def gen(s, c):
        hi = _lsr(torch, splitmix64(torch, seed, c, s, device), 32)  # 0 .. 2^32-1
        return (hi - ((hi >> 31) << 32)).to(torch.int32)             # same low 32 bits, in range
    return _chunked(torch, n, torch.int32, gen, device)


def c2_float32(torch, n, seed=2, device="cuda"):
    def gen(s, c):
        f = u01(torch, seed, c, s, device) * 2e6
        f = f + (-1e6)
        r = splitmix64(torch, seed + 1000, c, s, device)
        special = _umod(torch, r, 100) == 0
        kind = _lsr(torch, r, 8) % 4
        sign = (_lsr(torch, r, 16) & 1) << 31
        mant = (_lsr(torch, r, 20) % 0x7FFFFF) + 1
        bits = torch.where(kind == 0, torch.zeros_like(r),
                           torch.where(kind == 1, torch.full_like(r, 0x80000000), mant | sign))
        bits32 = (bits - ((bits >> 31) << 32)).to(torch.int32)
        fb = f.view(torch.int32).clone()
        fb[special] = bits32[special]
        return fb.view(torch.float32)
    return _chunked(torch, n, torch.float32, gen, device)


def c3_uint64(torch, n, kind, seed=3, device="cuda"):
    """int64 tensor with the bits of datagen.c3_uint64."""
    def gen(s, c):
        r = splitmix64(torch, seed, c, s, device)
        if kind == "full":
            return r
        if kind == "low16":
            return r & 0xFFFF
        if kind == "skew90":
            pick = _umod(torch, splitmix64(torch, seed + 1000, c, s, device), 10)
            return torch.where(pick != 0, torch.full_like(r, datagen.C3_CONSTANT), r)
        raise ValueError(kind)
    return _chunked(torch, n, torch.int64, gen, device)


def c4_segments(torch, n, mean, seed=4, device="cuda"):
    """(int32 keys = run index with run lengths ~ Geometric(1/mean), float32 values)."""
    nseg = int(n / mean * 1.2) + 1000
    r = splitmix64(torch, seed, nseg, 0, device)
    # (uint64 + 0.5) / 2^64 in float64, from the two halves so that no sign gets in the way
    u = (_lsr(torch, r, 11).to(torch.float64) + 0.5) / float(1 << 53)
    lens = (torch.floor(torch.log(u) / float(np.log1p(-1.0 / mean))) + 1).to(torch.int64)
    keys = torch.repeat_interleave(torch.arange(nseg, device=device, dtype=torch.int32), lens)[:n].contiguous()
    if keys.numel() != n:
        raise RuntimeError("config-4 generator came up short")
    vals = _chunked(torch, n, torch.float32, lambda s, c: u01(torch, seed + 1000, c, s, device), device)
    return keys, vals


def c5_float32(torch, n, seed=5, device="cuda"):
    return _chunked(torch, n, torch.float32, lambda s, c: u01(torch, seed, c, s, device), device)


def c5_merge_inputs(torch, n_each, seed=6, device="cuda"):
    """Two sorted uint32 arrays (as int32 bits) with payload = original index (int32)."""
    out = []
    for j in range(2):
        k = c2_uint32(torch, n_each, seed + j, device).to(torch.int64) & 0xFFFFFFFF
        ks, order = torch.sort(k, stable=True)
        out.append(((ks - ((ks >> 31) << 32)).to(torch.int32), order.to(torch.int32)))
    return out
