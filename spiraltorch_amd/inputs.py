"""Deterministic synthetic inputs shared by the tests and the benchmark.

splitmix64 keyed by (seed, element index), so any slice of a tensor can be generated without the rest:
  uniform: u = (x >> 40) · 2⁻²⁴ ∈ [0, 1);  value = lo + (hi − lo)·u  (evaluated in f32)
  normal:  Box–Muller on two draws per pair, evaluated in f64 and cast to f32
  bf16:    round-to-nearest-even on the f32 bit pattern
Seeds follow 0xC0FFEE00 + 16·config + tensor_index.
"""
from __future__ import annotations

import numpy as np

_GAMMA = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)


def seed_for(config: int, tensor_index: int) -> int:
    return 0xC0FFEE00 + 16 * config + tensor_index


def splitmix64(seed: int, count: int, offset: int = 0) -> np.ndarray:
    """Outputs offset .. offset+count-1 of the splitmix64 stream started at `seed`."""
    with np.errstate(over="ignore"):
        idx = np.arange(offset + 1, offset + count + 1, dtype=np.uint64)
        z = np.uint64(seed & 0xFFFFFFFFFFFFFFFF) + idx * _GAMMA
        z = (z ^ (z >> np.uint64(30))) * _M1
        z = (z ^ (z >> np.uint64(27))) * _M2
        return z ^ (z >> np.uint64(31))


def uniform(seed: int, count: int, lo: float = 0.0, hi: float = 1.0) -> np.ndarray:
    x = splitmix64(seed, count)
    u = (x >> np.uint64(40)).astype(np.float32) * np.float32(2.0 ** -24)
    return (np.float32(lo) + (np.float32(hi) - np.float32(lo)) * u).astype(np.float32)


def normal(seed: int, count: int, mean: float = 0.0, std: float = 1.0) -> np.ndarray:
    pairs = (count + 1) // 2
    x = splitmix64(seed, 2 * pairs)
    u1 = ((x[0::2] >> np.uint64(11)).astype(np.float64) + 1.0) * 2.0 ** -53  # (0, 1]
    u2 = (x[1::2] >> np.uint64(11)).astype(np.float64) * 2.0 ** -53          # [0, 1)
    r = np.sqrt(-2.0 * np.log(u1))
    out = np.empty(2 * pairs, dtype=np.float64)
    out[0::2] = r * np.cos(2.0 * np.pi * u2)
    out[1::2] = r * np.sin(2.0 * np.pi * u2)
    return (mean + std * out[:count]).astype(np.float32)


def tokens(seed: int, count: int, vocab: int) -> np.ndarray:
    """Token ids uniform over 0..vocab-1, as the f32 values the embedding layer takes."""
    return (splitmix64(seed, count) % np.uint64(vocab)).astype(np.float32)


def to_bf16(values: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even f32 -> bf16 bit patterns (uint16)."""
    u = np.ascontiguousarray(values, dtype=np.float32).view(np.uint32)
    rounded = (u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))) >> np.uint32(16)
    nan = (u & np.uint32(0x7FFFFFFF)) > np.uint32(0x7F800000)
    rounded = np.where(nan, (u >> np.uint32(16)) | np.uint32(0x40), rounded)
    return rounded.astype(np.uint16)


def from_bf16(bits: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(bits, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)
