"""Seeded synthetic inputs for the benchmark configurations.

Everything derives from the SplitMix64 stream ``x_i = mix(seed + (i+1) * GAMMA)``
so that any implementation (C#, C++, numpy) can regenerate the same arrays.
All functions are chunked numpy and return host arrays.
"""
from __future__ import annotations

import numpy as np

DEFAULT_SEED = 0x123456789ABCDEF0
_GAMMA = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)
_CHUNK = 1 << 22


def splitmix64(n: int, seed: int = DEFAULT_SEED, start: int = 0) -> np.ndarray:
    """x_start .. x_{start+n-1} of the SplitMix64 stream as uint64."""
    out = np.empty(n, dtype=np.uint64)
    with np.errstate(over="ignore"):
        for lo in range(0, n, _CHUNK):
            hi = min(n, lo + _CHUNK)
            i = np.arange(start + lo + 1, start + hi + 1, dtype=np.uint64)
            z = np.uint64(seed & 0xFFFFFFFFFFFFFFFF) + i * _GAMMA
            z = (z ^ (z >> np.uint64(30))) * _M1
            z = (z ^ (z >> np.uint64(27))) * _M2
            out[lo:hi] = z ^ (z >> np.uint64(31))
    return out


def _unit_float64(x: np.ndarray) -> np.ndarray:
    """53-bit uniform in [0, 1)."""
    return (x >> np.uint64(11)).astype(np.float64) * (1.0 / 9007199254740992.0)


def uniform_u32(n: int, seed: int = DEFAULT_SEED) -> np.ndarray:
    """Uniform keys over the full 32-bit range: low 32 bits of each draw."""
    return splitmix64(n, seed).astype(np.uint32)


def uniform_u64(n: int, seed: int = DEFAULT_SEED) -> np.ndarray:
    return splitmix64(n, seed)


def zipf_u32(n: int, s: float = 1.1, distinct: int = 1 << 16,
             seed: int = DEFAULT_SEED) -> np.ndarray:
    """Zipf(s) over ranks 0..distinct-1 by inverse CDF; the key is the rank."""
    w = 1.0 / np.power(np.arange(1, distinct + 1, dtype=np.float64), s)
    cdf = np.cumsum(w)
    cdf /= cdf[-1]
    out = np.empty(n, dtype=np.uint32)
    for lo in range(0, n, _CHUNK):
        hi = min(n, lo + _CHUNK)
        u = _unit_float64(splitmix64(hi - lo, seed, start=lo))
        out[lo:hi] = np.minimum(np.searchsorted(cdf, u, side="right"),
                                distinct - 1).astype(np.uint32)
    return out


def constant_u32(n: int, value: int = 0xDEADBEEF) -> np.ndarray:
    return np.full(n, value, dtype=np.uint32)


def small_ints_i32(n: int, seed: int = DEFAULT_SEED) -> np.ndarray:
    """int32 values uniform in [0, 15]."""
    return (splitmix64(n, seed) & np.uint64(15)).astype(np.int32)


def _box_muller(x0: np.ndarray, x1: np.ndarray) -> np.ndarray:
    u0 = 1.0 - _unit_float64(x0)  # (0, 1]
    u1 = _unit_float64(x1)
    return np.sqrt(-2.0 * np.log(u0)) * np.cos(2.0 * np.pi * u1)


def normal_f32(n: int, seed: int = DEFAULT_SEED) -> np.ndarray:
    """N(0,1) by Box-Muller in float64 from draws (2i, 2i+1), cast to float32."""
    out = np.empty(n, dtype=np.float32)
    for lo in range(0, n, _CHUNK):
        hi = min(n, lo + _CHUNK)
        x = splitmix64(2 * (hi - lo), seed, start=2 * lo)
        out[lo:hi] = _box_muller(x[0::2], x[1::2]).astype(np.float32)
    return out


def bytes_u8(n: int, seed: int = DEFAULT_SEED) -> np.ndarray:
    """Uniform bytes: byte j of draw i/8 (little endian)."""
    draws = splitmix64((n + 7) // 8, seed)
    return draws.view(np.uint8)[:n].copy()


def gaussian_mixture_i32(n: int, bins: int = 4096, components: int = 8,
                         sigma: float = 96.0,
                         seed: int = DEFAULT_SEED) -> np.ndarray:
    """Mixture of `components` Gaussians (means 256 + 512 j), clipped to
    [0, bins-1], as int32.  Draw 3i picks the component, draws 3i+1 and 3i+2
    feed Box-Muller."""
    out = np.empty(n, dtype=np.int32)
    for lo in range(0, n, _CHUNK):
        hi = min(n, lo + _CHUNK)
        x = splitmix64(3 * (hi - lo), seed, start=3 * lo)
        comp = (x[0::3] & np.uint64(components - 1)).astype(np.float64)
        z = _box_muller(x[1::3], x[2::3])
        v = np.rint(256.0 + 512.0 * comp + sigma * z)
        out[lo:hi] = np.clip(v, 0, bins - 1).astype(np.int32)
    return out


# ---- the same streams generated on the GPU (torch int64 arithmetic) ---------
# int64 multiplication and addition wrap like uint64, and a logical right shift
# is an arithmetic one followed by a mask, so the bits equal the numpy version.
def _as_i64(v: int) -> int:
    v &= 0xFFFFFFFFFFFFFFFF
    return v - (1 << 64) if v >= (1 << 63) else v


def splitmix64_torch(n: int, seed: int = DEFAULT_SEED, start: int = 0,
                     device: str = "cuda:0"):
    """x_start .. x_{start+n-1} as an int64 tensor holding the uint64 bits."""
    import torch

    def lsr(z, k):
        return (z >> k) & ((1 << (64 - k)) - 1)

    out = torch.empty(n, dtype=torch.int64, device=device)
    chunk = 1 << 26
    for lo in range(0, n, chunk):
        hi = min(n, lo + chunk)
        i = torch.arange(start + lo + 1, start + hi + 1, dtype=torch.int64,
                         device=device)
        z = i * _as_i64(int(_GAMMA)) + _as_i64(seed)
        z = (z ^ lsr(z, 30)) * _as_i64(int(_M1))
        z = (z ^ lsr(z, 27)) * _as_i64(int(_M2))
        out[lo:hi] = z ^ lsr(z, 31)
    return out


def _unit_float64_torch(x):
    import torch
    return ((x >> 11) & ((1 << 53) - 1)).to(torch.float64) * (1.0 / 9007199254740992.0)


def uniform_u32_torch(n: int, seed: int = DEFAULT_SEED, device: str = "cuda:0"):
    """Bits of uniform_u32 as an int32 tensor."""
    import torch
    return splitmix64_torch(n, seed, device=device).to(torch.int32)


def small_ints_i32_torch(n: int, seed: int = DEFAULT_SEED, device: str = "cuda:0"):
    import torch
    return (splitmix64_torch(n, seed, device=device) & 15).to(torch.int32)


def bytes_u8_torch(n: int, seed: int = DEFAULT_SEED, device: str = "cuda:0"):
    import torch
    return splitmix64_torch((n + 7) // 8, seed, device=device).view(torch.uint8)[:n]


def zipf_u32_torch(n: int, s: float = 1.1, distinct: int = 1 << 16,
                   seed: int = DEFAULT_SEED, device: str = "cuda:0"):
    """Bits of zipf_u32 as an int32 tensor (same table, same comparisons)."""
    import torch
    w = 1.0 / np.power(np.arange(1, distinct + 1, dtype=np.float64), s)
    cdf = np.cumsum(w)
    cdf /= cdf[-1]
    table = torch.from_numpy(cdf).to(device)
    out = torch.empty(n, dtype=torch.int32, device=device)
    chunk = 1 << 26
    for lo in range(0, n, chunk):
        hi = min(n, lo + chunk)
        u = _unit_float64_torch(splitmix64_torch(hi - lo, seed, start=lo, device=device))
        r = torch.searchsorted(table, u, right=True).clamp_(max=distinct - 1)
        out[lo:hi] = r.to(torch.int32)
    return out


def _box_muller_torch(x0, x1):
    import torch
    u0 = 1.0 - _unit_float64_torch(x0)
    u1 = _unit_float64_torch(x1)
    return torch.sqrt(-2.0 * torch.log(u0)) * torch.cos(2.0 * np.pi * u1)


def normal_f32_torch(n: int, seed: int = DEFAULT_SEED, device: str = "cuda:0"):
    """Same construction as normal_f32; log/cos may differ from numpy's in the
    last float64 bit, so equality with the host version is not guaranteed."""
    import torch
    out = torch.empty(n, dtype=torch.float32, device=device)
    chunk = 1 << 25
    for lo in range(0, n, chunk):
        hi = min(n, lo + chunk)
        x = splitmix64_torch(2 * (hi - lo), seed, start=2 * lo, device=device)
        out[lo:hi] = _box_muller_torch(x[0::2], x[1::2]).to(torch.float32)
    return out


def gaussian_mixture_i32_torch(n: int, bins: int = 4096, components: int = 8,
                               sigma: float = 96.0, seed: int = DEFAULT_SEED,
                               device: str = "cuda:0"):
    import torch
    out = torch.empty(n, dtype=torch.int32, device=device)
    chunk = 1 << 25
    for lo in range(0, n, chunk):
        hi = min(n, lo + chunk)
        x = splitmix64_torch(3 * (hi - lo), seed, start=3 * lo, device=device)
        comp = (x[0::3] & (components - 1)).to(torch.float64)
        z = _box_muller_torch(x[1::3], x[2::3])
        v = torch.round(256.0 + 512.0 * comp + sigma * z)
        out[lo:hi] = v.clamp_(0, bins - 1).to(torch.int32)
    return out
