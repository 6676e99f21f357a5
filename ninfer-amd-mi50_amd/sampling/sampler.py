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
from typing import Dict, Iterable, List, Optional, Sequence, Tuple

import numpy as np
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


class History:
    """How often a request has seen each token (prompt + generated), for the
    repetition penalty. Kept as two growing arrays (distinct tokens, counts), so
    that a step hands them to the device as they are: the work per generated
    token does not grow with the length of the history."""

    def __init__(self, tokens: Iterable[int] = ()):
        toks, counts = np.unique(np.asarray(list(tokens), dtype=np.int64), return_counts=True)
        n = int(toks.shape[0])
        cap = max(64, 2 * n)
        self._tok = np.zeros(cap, np.int32)
        self._cnt = np.zeros(cap, np.int32)
        self._tok[:n] = toks
        self._cnt[:n] = counts
        self._n = n
        self._where: Optional[Dict[int, int]] = None   # token -> index, made at the first add

    def add(self, token: int) -> None:
        if self._where is None:
            self._where = {int(t): i for i, t in enumerate(self._tok[:self._n])}
        i = self._where.get(token)
        if i is not None:
            self._cnt[i] += 1
            return
        if self._n == self._tok.shape[0]:
            self._tok = np.concatenate([self._tok, np.zeros_like(self._tok)])
            self._cnt = np.concatenate([self._cnt, np.zeros_like(self._cnt)])
        self._tok[self._n] = token
        self._cnt[self._n] = 1
        self._where[token] = self._n
        self._n += 1

    def arrays(self) -> Tuple[np.ndarray, np.ndarray]:
        """(distinct tokens, their counts), int32 views of equal length."""
        return self._tok[:self._n], self._cnt[:self._n]

    def count(self, token: int) -> int:
        toks, cnts = self.arrays()
        hit = np.nonzero(toks == token)[0]
        return int(cnts[hit[0]]) if hit.size else 0

    def __len__(self) -> int:
        return self._n


class SampleRow:
    """What the sampler needs of one row: options, history counts, RNG stream."""

    def __init__(self, params: SamplingParams, history: History, key: int, draw: int, seed: int):
        self.params = params
        self.history = history if isinstance(history, History) else History(
            t for t, c in dict(history).items() for _ in range(c))
        self.key = key
        self.draw = draw
        self.seed = seed


class Sampler:
    def __init__(self, ops, device):
        self.ops = ops
        self.device = device
        self._staging: List[list] = []   # pinned buffers (and the event after each one's copy)
        self._staging_next = 0

    def _to_device(self, packed: np.ndarray) -> torch.Tensor:
        """The rows' packed parameters on the device, through one of a few pinned buffers used in
        turn: the copy is queued behind the step that makes the logits and the host goes on (a
        copy out of pageable memory makes the host wait until the device has reached it, and the
        sampling kernel would then be launched only after the step has ended)."""
        host = torch.from_numpy(packed)
        if self.device.type != "cuda":
            return host.to(self.device)
        n = host.numel()
        if len(self._staging) < 4:
            self._staging.append([torch.empty(max(n, 1024), dtype=torch.int32).pin_memory(),
                                  torch.cuda.Event()])
            slot = self._staging[-1]
        else:
            slot = self._staging[self._staging_next]
            self._staging_next = (self._staging_next + 1) % len(self._staging)
            slot[1].synchronize()
            if slot[0].numel() < n:
                slot[0] = torch.empty(2 * n, dtype=torch.int32).pin_memory()
        slot[0][:n].copy_(host)
        dev = torch.empty(n, dtype=torch.int32, device=self.device)
        dev.copy_(slot[0][:n], non_blocking=True)
        slot[1].record()
        return dev

    def sample(self, logits: torch.Tensor, rows: Sequence[SampleRow]) -> List[int]:
        """One token per row of `logits` [R, vocab]."""
        r = len(rows)
        assert logits.shape[0] == r
        # Everything the kernel needs of the rows travels in one array and one copy: four
        # 32-bit floats and one int per row, the offsets of the penalties, then their tokens
        # and counts. (Copies queue behind the step that makes the logits, one after the other:
        # every further one would add its latency to the step.)
        pen_t: List[np.ndarray] = []
        pen_c: List[np.ndarray] = []
        pen_o = np.zeros(r + 1, np.int32)
        for i, row in enumerate(rows):
            n = 0
            if row.params.repetition_penalty != 1.0:
                toks, cnts = row.history.arrays()
                pen_t.append(toks)
                pen_c.append(cnts)
                n = toks.shape[0]
            pen_o[i + 1] = pen_o[i] + n
        floats = np.empty((4, r), np.float32)
        floats[0] = [row.params.temperature for row in rows]
        floats[1] = [row.params.top_p for row in rows]
        floats[2] = [row.params.repetition_penalty for row in rows]
        floats[3] = [uniform(row.seed, row.key, row.draw) for row in rows]
        top_k = np.asarray([row.params.top_k for row in rows], np.int32)
        n_pen = int(pen_o[-1])
        packed = np.concatenate([floats.reshape(-1).view(np.int32), top_k, pen_o] + pen_t + pen_c)
        dev = self._to_device(packed)
        f = dev[:4 * r].view(torch.float32)
        o = 4 * r
        pen = {}
        if n_pen > 0:
            pen = dict(pen_offsets=dev[o + r:o + 2 * r + 1],
                       pen_tokens=dev[o + 2 * r + 1:o + 2 * r + 1 + n_pen],
                       pen_counts=dev[o + 2 * r + 1 + n_pen:o + 2 * r + 1 + 2 * n_pen])
        out = torch.empty(r, dtype=torch.int32, device=self.device)
        # rows that are greedy or keep at most a few dozen tokens (the reference's default is
        # top_k = 50) take the path that reads the logits with the whole GPU
        most = getattr(self.ops, "FEW_TOKENS", 0)
        # (rows that are all greedy stay with the one launch: it is short as it is)
        if most and any(row.params.temperature > 0 for row in rows) and all(
                row.params.temperature <= 0 or 1 <= row.params.top_k <= most for row in rows):
            pen["few"] = True
        self.ops.sample(logits, f[:r], f[3 * r:4 * r], out, top_k=dev[o:o + r], top_p=f[r:2 * r],
                        rep_penalty=f[2 * r:3 * r], **pen)
        return out.tolist()
