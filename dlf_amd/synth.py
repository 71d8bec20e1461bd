"""Seeded synthetic inputs of the benchmark configurations, generated with torch
ops so the same code fills host or device memory.

Counter-based: element i of a stream is splitmix64(seed, i), so any slice can
be regenerated independently and in chunks.  Normals come from Box-Muller in
fp64 and are then cast.
"""
from __future__ import annotations

import math

import torch

_GOLD = 0x9E3779B97F4A7C15 - (1 << 64)      # as signed 64-bit
_M1 = 0xBF58476D1CE4E5B9 - (1 << 64)
_M2 = 0x94D049BB133111EB - (1 << 64)
_SEED_MUL = 0xD1B54A32D192ED03


def _lsr(x: torch.Tensor, s: int) -> torch.Tensor:
    return (x >> s) & ((1 << (64 - s)) - 1)


def _signed(v: int) -> int:
    v &= (1 << 64) - 1
    return v - (1 << 64) if v >= (1 << 63) else v


def splitmix64(seed: int, index: torch.Tensor) -> torch.Tensor:
    """index: int64 tensor of counters -> int64 tensor holding the 64 random bits."""
    z = (index + 1) * _GOLD + _signed(seed * _SEED_MUL)
    z = (z ^ _lsr(z, 30)) * _M1
    z = (z ^ _lsr(z, 27)) * _M2
    return z ^ _lsr(z, 31)


def _chunks(count: int, chunk: int):
    for lo in range(0, count, chunk):
        yield lo, min(count, lo + chunk)


def fill(out: torch.Tensor, fn, chunk: int = 1 << 24) -> torch.Tensor:
    """out.view(-1)[lo:hi] = fn(arange(lo, hi)) chunk by chunk (bounded temporaries)."""
    flat = out.view(-1)
    for lo, hi in _chunks(flat.numel(), chunk):
        idx = torch.arange(lo, hi, dtype=torch.int64, device=out.device)
        flat[lo:hi] = fn(idx).to(out.dtype)
    return out


def uniform01(seed: int):
    return lambda idx: _lsr(splitmix64(seed, idx), 11).to(torch.float64) * (1.0 / (1 << 53))


def normal(seed: int):
    def fn(idx):
        u1 = (_lsr(splitmix64(seed, 2 * idx), 11).to(torch.float64) + 1.0) * (1.0 / (1 << 53))
        u2 = _lsr(splitmix64(seed, 2 * idx + 1), 11).to(torch.float64) * (1.0 / (1 << 53))
        return torch.sqrt(-2.0 * torch.log(u1)) * torch.cos((2.0 * math.pi) * u2)
    return fn


def randint(seed: int, lo: int, hi: int):
    return lambda idx: (_lsr(splitmix64(seed, idx), 1) % (hi - lo)) + lo


def full_range_i64(seed: int):
    return lambda idx: splitmix64(seed, idx)


def unit_interval_exact(seed: int):
    """x = u24 * 2^-23 - 1 in U(-1, 1): exactly representable in fp32, so sums are exact in fp64."""
    return lambda idx: (_lsr(splitmix64(seed, idx), 40).to(torch.float64) * (1.0 / (1 << 23))) - 1.0


def quantised_normal(seed: int, sigma: float = 2.0, steps: int = 256):
    n = normal(seed)
    return lambda idx: torch.round(n(idx) * (sigma * steps)) / steps


def quantised_uniform(seed: int, levels: int = 4096):
    u = uniform01(seed)
    return lambda idx: torch.floor(u(idx) * levels) / levels
