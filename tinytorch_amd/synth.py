"""Synthetic inputs: a counter-based normal generator that runs on the device.

Element i of a draw depends only on (seed, stream, i): a splitmix64 finaliser over a counter gives two uniforms,
Box-Muller in float64 gives the normal, which is scaled and rounded to float32.  Benchmarks draw their Q / K / V from
it (fixed seeds, one stream per tensor) instead of the framework's own generator, whose stream is not portable.
The arithmetic is written with torch integer ops so that it runs where the tensors live; log and cos are the
device's, so a value may differ from another implementation of the same recipe in the last bit.
"""
import torch

_M64 = (1 << 64) - 1
_GOLD = 0x9E3779B97F4A7C15
_C1 = 0xBF58476D1CE4E5B9
_C2 = 0x94D049BB133111EB


def _s64(x):
    """Python integer (mod 2^64) as the int64 with the same bits."""
    x &= _M64
    return x - (1 << 64) if x >> 63 else x


def _mix64_int(z):
    z = (z + _GOLD) & _M64
    z = ((z ^ (z >> 30)) * _C1) & _M64
    z = ((z ^ (z >> 27)) * _C2) & _M64
    return z ^ (z >> 31)


def _lshr(x, k):
    """Logical right shift of int64 tensors (torch's >> is arithmetic)."""
    return (x >> k) & ((1 << (64 - k)) - 1)


def _mix64(z):
    z = z + _s64(_GOLD)
    z = (z ^ _lshr(z, 30)) * _s64(_C1)
    z = (z ^ _lshr(z, 27)) * _s64(_C2)
    return z ^ _lshr(z, 31)


def randn(seed, stream, shape, mul=1.0, device="cuda", chunk=1 << 24):
    """float32 tensor of `shape` on `device`: i.i.d. N(0, 1) * mul from (seed, stream)."""
    n = 1
    for d in shape:
        n *= int(d)
    key = _mix64_int((seed & _M64) ^ _mix64_int((stream * 0xD1342543DE82EF95 + 0x632BE59BD9B4E019) & _M64))
    out = torch.empty(n, dtype=torch.float32, device=device)
    for lo in range(0, n, chunk):
        hi = min(n, lo + chunk)
        i = torch.arange(lo, hi, dtype=torch.int64, device=device)
        ctr = i * 2 + _s64(key)
        a = _mix64(ctr)
        b = _mix64(ctr + 1)
        u1 = (_lshr(a, 11).double() + 1.0) * 2.0 ** -53  # (0, 1]
        u2 = _lshr(b, 11).double() * 2.0 ** -53          # [0, 1)
        z = torch.sqrt(-2.0 * torch.log(u1)) * torch.cos(6.283185307179586476925286766559 * u2)
        out[lo:hi] = (float(mul) * z).float()
    return out.reshape(tuple(shape))
