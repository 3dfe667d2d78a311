"""Deterministic synthetic inputs: a counter-based generator (splitmix64 on the
element index) evaluated with torch integer ops, so the same code produces the
same stream on the CPU and on the GPU and fixtures never depend on a library's
RNG implementation."""
import math

import torch

_M64 = (1 << 64) - 1


def _s64(v):
    """Python int -> the int64 with the same low 64 bits."""
    v &= _M64
    return v - (1 << 64) if v >= (1 << 63) else v


def _lsr(x, n):
    """Logical right shift of an int64 tensor."""
    return (x >> n) & ((1 << (64 - n)) - 1)


def _splitmix64(idx, seed):
    z = idx * _s64(0x9E3779B97F4A7C15) + _s64(seed * 0xD1342543DE82EF95 + 0x632BE59BD9B4E019)
    z = (z ^ _lsr(z, 30)) * _s64(0xBF58476D1CE4E5B9)
    z = (z ^ _lsr(z, 27)) * _s64(0x94D049BB133111EB)
    return z ^ _lsr(z, 31)


def _unit(bits):
    """24 high bits -> float32 in [0, 1)."""
    return (_lsr(bits, 40).to(torch.float32)) * (1.0 / 16777216.0)


def uniform(shape, seed, lo=-1.0, hi=1.0, device="cpu"):
    n = math.prod(shape)
    idx = torch.arange(n, dtype=torch.int64, device=device)
    u = _unit(_splitmix64(idx, seed))
    return (lo + (hi - lo) * u).reshape(shape)


def normal(shape, seed, std=1.0, device="cpu"):
    """Box-Muller on two independent counter streams."""
    n = math.prod(shape)
    idx = torch.arange(n, dtype=torch.int64, device=device)
    u1 = _unit(_splitmix64(2 * idx, seed))
    u2 = _unit(_splitmix64(2 * idx + 1, seed))
    r = torch.sqrt(-2.0 * torch.log(1.0 - u1))  # 1 - u1 in (0, 1]
    return (std * r * torch.cos((2.0 * math.pi) * u2)).reshape(shape)
