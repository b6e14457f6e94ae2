"""Counter-based pseudo-random inputs: splitmix64 of (seed, element index).

One generator for benchmark inputs (on the GPU, with torch integer ops) and test inputs
(on the host, with numpy): element i of stream `seed` is the same 64-bit word on either
side, whatever the order or the device it is drawn on.  The reference's own tests draw
from glibc rand() seeded by the clock (ark/unittest/unittest_utils.h:54-56), which cannot
be reproduced; a counter-based generator can.

Uniforms take the word's top 24 bits (exact in fp32).  Normals are Box-Muller over two
words; their last fp32 bit depends on the platform's log/cos, so a consumer that needs the
same bits on both sides generates once and copies.
"""
import math

_GOLD = 0x9E3779B97F4A7C15
_M1 = 0xBF58476D1CE4E5B9
_M2 = 0x94D049BB133111EB


def _s64(v):
    """The two's-complement int64 with the bits of the unsigned 64-bit `v`."""
    v &= (1 << 64) - 1
    return v - (1 << 64) if v >> 63 else v


def _words_numpy(seed, start, count):
    import numpy as np
    with np.errstate(over="ignore"):
        z = np.arange(start, start + count, dtype=np.uint64)
        z = z + np.uint64((seed * _GOLD + _GOLD) & ((1 << 64) - 1))
        z = (z ^ (z >> np.uint64(30))) * np.uint64(_M1)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(_M2)
        return z ^ (z >> np.uint64(31))


def _words_torch(seed, start, count, device):
    import torch

    def lsr(x, s):  # logical shift right on int64
        return (x >> s) & ((1 << (64 - s)) - 1)

    z = torch.arange(start, start + count, dtype=torch.int64, device=device)
    z = z + _s64(seed * _GOLD + _GOLD)
    z = (z ^ lsr(z, 30)) * _s64(_M1)
    z = (z ^ lsr(z, 27)) * _s64(_M2)
    return z ^ lsr(z, 31)


def uniform(seed, shape, lo=0.0, hi=1.0, device=None):
    """fp32 values in [lo, hi): numpy array (device None) or torch tensor on `device`."""
    n = int(math.prod(shape))
    if device is None:
        import numpy as np
        u = (_words_numpy(seed, 0, n) >> np.uint64(40)).astype(np.float32) * np.float32(2.0 ** -24)
        return (np.float32(lo) + u * np.float32(hi - lo)).reshape(shape)
    import torch
    w = _words_torch(seed, 0, n, device)
    u = ((w >> 40) & ((1 << 24) - 1)).to(torch.float32) * (2.0 ** -24)
    return (lo + u * (hi - lo)).reshape(shape)


def normal(seed, shape, mean=0.0, std=1.0, device=None):
    """fp32 N(mean, std^2) by Box-Muller over two words per value."""
    n = int(math.prod(shape))
    if device is None:
        import numpy as np
        w1, w2 = _words_numpy(seed, 0, n), _words_numpy(seed, n, n)
        u1 = ((w1 >> np.uint64(40)).astype(np.float32) + np.float32(1.0)) * np.float32(2.0 ** -24)  # (0, 1]
        u2 = (w2 >> np.uint64(40)).astype(np.float32) * np.float32(2.0 ** -24)
        z = np.sqrt(np.float32(-2.0) * np.log(u1)) * np.cos(np.float32(2.0 * math.pi) * u2)
        return (np.float32(mean) + np.float32(std) * z).astype(np.float32).reshape(shape)
    import torch
    w1, w2 = _words_torch(seed, 0, n, device), _words_torch(seed, n, n, device)
    u1 = (((w1 >> 40) & ((1 << 24) - 1)).to(torch.float32) + 1.0) * (2.0 ** -24)
    u2 = ((w2 >> 40) & ((1 << 24) - 1)).to(torch.float32) * (2.0 ** -24)
    z = torch.sqrt(-2.0 * torch.log(u1)) * torch.cos((2.0 * math.pi) * u2)
    return (mean + std * z).reshape(shape)


def seed_of(config, tensor_name):
    """A stable 31-bit seed per (configuration, tensor name)."""
    h = 1469598103934665603
    for ch in f"{config}/{tensor_name}".encode():
        h = ((h ^ ch) * 1099511628211) & ((1 << 64) - 1)
    return h & 0x7FFFFFFF
