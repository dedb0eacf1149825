"""Seeded synthetic inputs that are bit-reproducible on any host.

The reference draws test tensors from libstdc++'s ``std::mt19937`` +
``std::normal_distribution`` (paperkiln tests/test_gradcheck.cpp:32-39), whose
stream depends on the C++ library. Parity across machines needs a generator
this repo owns: splitmix64 for the bits and Box-Muller for the normals, both
evaluated in numpy float64 and rounded once to fp32.
"""
from __future__ import annotations

import numpy as np

_MASK = np.uint64(0xFFFFFFFFFFFFFFFF)


def splitmix64(seed: int, n: int) -> np.ndarray:
    """n successive outputs of splitmix64 started at ``seed`` (uint64)."""
    with np.errstate(over="ignore"):
        idx = np.arange(1, n + 1, dtype=np.uint64)
        z = (np.uint64(seed & 0xFFFFFFFFFFFFFFFF) + idx * np.uint64(0x9E3779B97F4A7C15)) & _MASK
        z = ((z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)) & _MASK
        z = ((z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)) & _MASK
        return z ^ (z >> np.uint64(31))


def uniform01(seed: int, n: int) -> np.ndarray:
    """n doubles in (0, 1): top 53 bits, offset by half an ulp so 0 is excluded."""
    return ((splitmix64(seed, n) >> np.uint64(11)).astype(np.float64) + 0.5) * (1.0 / (1 << 53))


def randn(seed: int, shape, std: float = 1.0) -> np.ndarray:
    """i.i.d. N(0, std^2) fp32 tensor of ``shape`` via Box-Muller."""
    n = int(np.prod(shape))
    m = (n + 1) // 2
    u = uniform01(seed, 2 * m)
    r = np.sqrt(-2.0 * np.log(u[:m]))
    th = 2.0 * np.pi * u[m:]
    out = np.empty(2 * m, dtype=np.float64)
    out[0::2] = r * np.cos(th)
    out[1::2] = r * np.sin(th)
    return (out[:n] * std).astype(np.float32).reshape(shape)


def randint(seed: int, n: int, hi: int) -> np.ndarray:
    """n int32 ids uniform over [0, hi)."""
    return (splitmix64(seed, n) % np.uint64(hi)).astype(np.int32)


def bf16_round(x: np.ndarray) -> np.ndarray:
    """Round fp32 to the nearest bf16 (ties to even), returned as fp32."""
    b = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    r = ((b >> np.uint32(16)) & np.uint32(1)) + np.uint32(0x7FFF)
    return ((b + r) & np.uint32(0xFFFF0000)).view(np.float32)


def to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """fp32 -> bf16 bit patterns (uint16), round to nearest even."""
    return (bf16_round(x).view(np.uint32) >> np.uint32(16)).astype(np.uint16)


def from_bf16_bits(b: np.ndarray) -> np.ndarray:
    return (b.astype(np.uint32) << np.uint32(16)).view(np.float32)


def rope_interleaved(x: np.ndarray, theta: float) -> np.ndarray:
    """RoPE on adjacent pairs (x[2j], x[2j+1]) of every head of a
    [B,T,H,dk] tensor, positions 0..T-1 per sequence, evaluated in fp32 with
    the reference's formula (paperkiln src/ops.cpp:497-509). Input prep for the
    "RoPE pre-applied" workloads; unlike the reference op it rotates every head.
    """
    B, T, H, dk = x.shape
    dim = np.arange(0, dk, 2, dtype=np.float32)
    inv = (np.float32(1.0) / np.power(np.float32(theta), dim / np.float32(dk))).astype(np.float32)
    ang = (np.arange(T, dtype=np.float32)[:, None] * inv[None, :]).astype(np.float32)
    c = np.cos(ang).astype(np.float32)[None, :, None, :]
    s = np.sin(ang).astype(np.float32)[None, :, None, :]
    x0, x1 = x[..., 0::2], x[..., 1::2]
    out = np.empty_like(x)
    out[..., 0::2] = x0 * c - x1 * s
    out[..., 1::2] = x0 * s + x1 * c
    return out


def visible_pairs(T: int, causal: bool, window: int, sinks: int) -> int:
    """Visible (query, key) pairs per head: the work model's unit."""
    if not causal:
        return T * T
    if window <= 0:
        return T * (T + 1) // 2
    i = np.arange(T, dtype=np.int64)
    win = np.minimum(i + 1, window)
    snk = np.minimum(sinks, np.maximum(0, i + 1 - window))
    return int((win + snk).sum())
