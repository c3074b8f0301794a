"""Deterministic synthetic inputs shared by the tests and the golden-vector
script.  Integer-only generation (splitmix64 + a 12-term Irwin-Hall sum), so
the same seed gives the same bits on every host and numpy version; values are
~N(0,1) and exactly representable in fp32 before the optional bf16 rounding.
"""
from __future__ import annotations

import numpy as np

_M64 = np.uint64(0xFFFFFFFFFFFFFFFF)


def _splitmix64(x: np.ndarray) -> np.ndarray:
    with np.errstate(over="ignore"):
        x = (x + np.uint64(0x9E3779B97F4A7C15)) & _M64
        z = x
        z = ((z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)) & _M64
        z = ((z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)) & _M64
        return z ^ (z >> np.uint64(31))


def u64(seed: int, n: int) -> np.ndarray:
    with np.errstate(over="ignore"):
        ctr = np.arange(n, dtype=np.uint64) * np.uint64(0xD1342543DE82EF95) + np.uint64(seed * 0x2545F4914F6CDD1D & 0xFFFFFFFFFFFFFFFF)
    return _splitmix64(ctr)


def normal_f32(seed: int, shape) -> np.ndarray:
    """~N(0,1): sum of twelve 16-bit uniforms, centred, scaled by 2^-16."""
    n = int(np.prod(shape))
    acc = np.zeros(n, np.int64)
    for part in range(3):
        w = u64(seed * 3 + part + 1, n)
        for s in range(4):
            acc += ((w >> np.uint64(16 * s)) & np.uint64(0xFFFF)).astype(np.int64)
    x = (acc - 6 * 65535).astype(np.float64) / 65536.0
    return x.astype(np.float32).reshape(shape)


def bf16_round_bits(x: np.ndarray) -> np.ndarray:
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    return ((u + np.uint64(0x7FFF) + ((u >> np.uint64(16)) & np.uint64(1))) >> np.uint64(16)).astype(np.uint16)


def bf16_widen(bits: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(bits, np.uint16).astype(np.uint32) << 16).view(np.float32)


def normal_bf16_bits(seed: int, shape) -> np.ndarray:
    return bf16_round_bits(normal_f32(seed, shape))


def normal_bf16_as_f32(seed: int, shape) -> np.ndarray:
    return bf16_widen(normal_bf16_bits(seed, shape))


def ints(seed: int, n: int, lo: int, hi: int) -> np.ndarray:
    """n integers uniform in [lo, hi] (inclusive)."""
    return (lo + (u64(seed, n) % np.uint64(hi - lo + 1)).astype(np.int64)).astype(np.int64)


def permutation(seed: int, n: int) -> np.ndarray:
    return np.argsort(u64(seed, n), kind="stable").astype(np.int32)


def ragged_lengths(seed: int, n_req: int, lo_tokens: int, hi_tokens: int, block: int = 128) -> np.ndarray:
    """Context lengths uniform in [lo, hi] rounded to the block size, as block counts."""
    return ints(seed, n_req, lo_tokens // block, hi_tokens // block).astype(np.int32)
