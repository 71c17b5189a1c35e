"""Counter-based synthetic data for the benchmark: element i of a stream is a pure function of
(seed, i), so any element of a matrix generated on the device can be recomputed on the host.

    z_i = splitmix64_finalizer((i + 1) * GOLDEN + seed * SEED_MUL)

    uniform [-1, 1):  2 * (top 24 bits of z) * 2^-24 - 1                      (exact in fp32)
    int8:             top 8 bits of z as a signed byte
    normal(mu, sd):   Box-Muller on u1 = ((bits 40..63) + 1) * 2^-24 in (0, 1] and
                      u2 = (bits 16..39) * 2^-24 in [0, 1): mu + sd * sqrt(-2 ln u1) * cos(2 pi u2),
                      evaluated in fp32

`*_device` build torch tensors on the GPU with integer tensor arithmetic (int64 wraps like
uint64), `*_host` are the numpy twins for any index array.  Uniform and int8 streams agree bit
for bit between the two; normals agree to the last bits of the device's and numpy's log / cos.
"""
from __future__ import annotations

import numpy as np

GOLDEN = 0x9E3779B97F4A7C15
SEED_MUL = 0xD1B54A32D192ED03
M1 = 0xBF58476D1CE4E5B9
M2 = 0x94D049BB133111EB
_CHUNK = 1 << 27  # elements generated at a time on the device (bounds the int64 temporaries)


def _s64(c: int) -> int:
    """A 64-bit constant as the signed value torch's int64 holds."""
    c &= (1 << 64) - 1
    return c - (1 << 64) if c >= (1 << 63) else c


# ---- host (numpy, uint64) ------------------------------------------------------------------
def bits_host(seed: int, idx) -> np.ndarray:
    idx = np.asarray(idx, dtype=np.uint64)
    with np.errstate(over="ignore"):
        z = (idx + np.uint64(1)) * np.uint64(GOLDEN) + np.uint64((seed * SEED_MUL) & ((1 << 64) - 1))
        z = (z ^ (z >> np.uint64(30))) * np.uint64(M1)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(M2)
        z = z ^ (z >> np.uint64(31))
    return z


def uniform_host(seed: int, idx) -> np.ndarray:
    z = bits_host(seed, idx)
    u = (z >> np.uint64(40)).astype(np.float32) * np.float32(2.0 ** -24)
    return (u * np.float32(2.0) - np.float32(1.0)).astype(np.float32)


def int8_host(seed: int, idx) -> np.ndarray:
    return (bits_host(seed, idx) >> np.uint64(56)).astype(np.uint8).view(np.int8)


def normal_host(seed: int, idx, mean: float = 0.0, std: float = 1.0) -> np.ndarray:
    z = bits_host(seed, idx)
    u1 = ((z >> np.uint64(40)).astype(np.float32) + np.float32(1.0)) * np.float32(2.0 ** -24)
    u2 = ((z >> np.uint64(16)) & np.uint64(0xFFFFFF)).astype(np.float32) * np.float32(2.0 ** -24)
    r = np.sqrt(np.float32(-2.0) * np.log(u1)).astype(np.float32)
    n = r * np.cos(np.float32(2.0 * np.pi) * u2).astype(np.float32)
    return (np.float32(mean) + np.float32(std) * n).astype(np.float32)


# ---- device (torch, int64 with wrap-around) -------------------------------------------------
def _lsr(z, k: int):
    return (z >> k) & ((1 << (64 - k)) - 1)


def _bits_device(seed: int, start: int, n: int, device):
    import torch
    i = torch.arange(start + 1, start + 1 + n, dtype=torch.int64, device=device)
    z = i * _s64(GOLDEN) + _s64(seed * SEED_MUL)
    z = (z ^ _lsr(z, 30)) * _s64(M1)
    z = (z ^ _lsr(z, 27)) * _s64(M2)
    return z ^ _lsr(z, 31)


def _chunks(n: int):
    for s in range(0, n, _CHUNK):
        yield s, min(_CHUNK, n - s)


def uniform_device(seed: int, n: int, device="cuda"):
    import torch
    out = torch.empty(n, dtype=torch.float32, device=device)
    for s, m in _chunks(n):
        z = _bits_device(seed, s, m, device)
        out[s:s + m] = _lsr(z, 40).to(torch.float32).mul_(2.0 ** -24).mul_(2.0).sub_(1.0)
    return out


def int8_device(seed: int, n: int, device="cuda"):
    import torch
    out = torch.empty(n, dtype=torch.int8, device=device)
    for s, m in _chunks(n):
        z = _bits_device(seed, s, m, device)
        out[s:s + m] = _lsr(z, 56).to(torch.uint8).view(torch.int8)
    return out


def normal_device(seed: int, n: int, mean: float = 0.0, std: float = 1.0, device="cuda"):
    import math

    import torch
    out = torch.empty(n, dtype=torch.float32, device=device)
    for s, m in _chunks(n):
        z = _bits_device(seed, s, m, device)
        u1 = _lsr(z, 40).to(torch.float32).add_(1.0).mul_(2.0 ** -24)
        u2 = (_lsr(z, 16) & 0xFFFFFF).to(torch.float32).mul_(2.0 ** -24)
        del z
        r = u1.log_().mul_(-2.0).sqrt_()
        r.mul_(u2.mul_(float(np.float32(2.0 * math.pi))).cos_())
        if std != 1.0:
            r.mul_(float(np.float32(std)))
        if mean != 0.0:
            r.add_(float(np.float32(mean)))
        out[s:s + m] = r
    return out
