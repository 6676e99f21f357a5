"""Seeded random numbers as a pure function of (key, index): the host mirror of
the device's fill kernel (csrc/fill.hip), bit for bit.

key = the first 8 bytes of sha256("<seed>:<tensor name>"). Element i hashes the
counters 3i, 3i + 1, 3i + 2 with splitmix64's finalizer over key + counter *
0x9E3779B97F4A7C15; the twelve 16-bit fields of the three hashes are added up
and z = (sum - 6 * 65535) / 65536: the sum of twelve uniform numbers, mean 0,
standard deviation 1 up to 1e-10, cut at +-6. Only integer arithmetic and one
exact conversion: host and device give the same bits. value = mean + std * z,
each operation rounded once to 32-bit.
"""
from __future__ import annotations

import hashlib

import numpy as np
import torch

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)


def tensor_key(seed: int, name: str) -> int:
    digest = hashlib.sha256(f"{int(seed)}:{name}".encode("utf-8")).digest()
    return int.from_bytes(digest[:8], "little")


def _mix64(z: np.ndarray) -> np.ndarray:
    z = (z ^ (z >> np.uint64(30))) * _M1
    z = (z ^ (z >> np.uint64(27))) * _M2
    return z ^ (z >> np.uint64(31))


def counter_normal(key: int, start: int, count: int) -> np.ndarray:
    """z(key, i) for i in [start, start + count), 32-bit."""
    with np.errstate(over="ignore"):
        i = np.arange(start, start + count, dtype=np.uint64)
        total = np.zeros(count, dtype=np.int64)
        for j in range(3):
            h = _mix64(np.uint64(key) + (np.uint64(3) * i + np.uint64(j)) * _GOLDEN)
            for shift in (0, 16, 32, 48):
                total += ((h >> np.uint64(shift)) & np.uint64(0xFFFF)).astype(np.int64)
    return (total - 6 * 65535).astype(np.float32) * np.float32(1.0 / 65536.0)


def fill(shape, key: int, std: float, mean: float = 0.0, chunk: int = 1 << 22) -> torch.Tensor:
    """A 32-bit tensor of the given shape: mean + std * z(key, flat index)."""
    n = 1
    for d in shape:
        n *= int(d)
    out = np.empty(n, dtype=np.float32)
    for start in range(0, n, chunk):
        z = counter_normal(key, start, min(chunk, n - start))
        out[start:start + z.size] = np.float32(mean) + np.float32(std) * z
    return torch.from_numpy(out).reshape(tuple(shape))
