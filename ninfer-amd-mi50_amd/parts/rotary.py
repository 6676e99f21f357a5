"""Rotary position encoding; half-split pairing (i, i + rot_dim/2) unless told
`pairing="interleaved"` (neighbours 2i, 2i + 1).

f_i = theta^(-2i/rot_dim), evaluated in double and rounded once to 32-bit
(reference src/models/model.hip:635-642 builds the same table with std::pow);
the angle pos * f_i, its sine and cosine and the rotation are 32-bit in the
kernel (reference src/ops/kernels.hip:73-94). `rot_dim` may be smaller than
the head size (the rest of the head is left alone); 0 means no rotation.
"""
from __future__ import annotations

import math
from typing import Optional

import torch

from ..registry import register_part
from .base import PositionEncoding, WeightBinder


class Rotary(PositionEncoding):
    def __init__(self, rot_dim: int, theta: float, pairing: str = "half"):
        if rot_dim % 2:
            raise ValueError(f"rotary dimension must be even, got {rot_dim}")
        if pairing not in ("half", "interleaved"):
            raise ValueError(f"pairing must be 'half' or 'interleaved', got {pairing!r}")
        self.rot_dim = rot_dim
        self.pairing = pairing
        self.theta = float(theta)
        self._table: Optional[torch.Tensor] = None

    def inv_freq(self) -> torch.Tensor:
        vals = [math.pow(self.theta, -(2.0 * i) / self.rot_dim)
                for i in range(self.rot_dim // 2)]
        return torch.tensor(vals, dtype=torch.float64).to(torch.float32)

    def bind(self, w: WeightBinder) -> None:
        self._table = self.inv_freq().to(w.device)

    def table(self) -> Optional[torch.Tensor]:
        return self._table


class NoPosition(PositionEncoding):
    """Queries and keys are used as projected."""
    rot_dim = 0

    def table(self) -> Optional[torch.Tensor]:
        return None


register_part("position", "rotary", Rotary)
register_part("position", "none", NoPosition)
