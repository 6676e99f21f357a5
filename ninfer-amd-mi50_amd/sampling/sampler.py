"""Sampling of next tokens from logits rows on the device.

Policy as the reference's `sample_logits` (src/runtime/engine.cpp:18-82):
repetition penalty over prompt + generated tokens, greedy if temperature
<= 0, else temperature, top-k, softmax, top-p, one draw. The reference seeds
`mt19937_64(seed + step)` per step (:166-169); here the uniform number of a
draw is a counter hash of (seed, request key, draw index), so a request's
tokens do not depend on what it was batched with. Seed 0 means "not fixed":
the request gets a seed from the operating system when it is added.
"""
from __future__ import annotations

import os
from collections import Counter
from typing import List, Sequence

import torch

from .params import SamplingParams

_MASK = (1 << 64) - 1


def _splitmix64(x: int) -> int:
    x = (x + 0x9E3779B97F4A7C15) & _MASK
    x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & _MASK
    return x ^ (x >> 31)


def uniform(seed: int, key: int, draw: int) -> float:
    """A number in [0, 1) with 24 random bits from (seed, key, draw)."""
    h = _splitmix64(_splitmix64(_splitmix64(seed & _MASK) ^ (key & _MASK)) ^ (draw & _MASK))
    return (h >> 40) / float(1 << 24)


def fresh_seed() -> int:
    return int.from_bytes(os.urandom(8), "little") | 1


class SampleRow:
    """What the sampler needs of one row: options, history counts, RNG stream."""

    def __init__(self, params: SamplingParams, history: Counter, key: int, draw: int, seed: int):
        self.params = params
        self.history = history
        self.key = key
        self.draw = draw
        self.seed = seed


class Sampler:
    def __init__(self, ops, device):
        self.ops = ops
        self.device = device

    def sample(self, logits: torch.Tensor, rows: Sequence[SampleRow]) -> List[int]:
        """One token per row of `logits` [R, vocab]."""
        r = len(rows)
        assert logits.shape[0] == r
        temp = [row.params.temperature for row in rows]
        top_k = [row.params.top_k for row in rows]
        top_p = [row.params.top_p for row in rows]
        rp = [row.params.repetition_penalty for row in rows]
        u = [uniform(row.seed, row.key, row.draw) for row in rows]
        pen_t: List[int] = []
        pen_c: List[int] = []
        pen_o = [0]
        for row in rows:
            if row.params.repetition_penalty != 1.0:
                for tok, cnt in row.history.items():
                    pen_t.append(tok)
                    pen_c.append(cnt)
            pen_o.append(len(pen_t))
        dev = self.device
        f32 = lambda v: torch.tensor(v, dtype=torch.float32, device=dev)
        i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)
        out = torch.empty(r, dtype=torch.int32, device=dev)
        pen = dict(pen_tokens=i32(pen_t), pen_counts=i32(pen_c), pen_offsets=i32(pen_o)) \
            if pen_t else {}
        self.ops.sample(logits, f32(temp), f32(u), out, top_k=i32(top_k), top_p=f32(top_p),
                        rep_penalty=f32(rp), **pen)
        return out.tolist()
