"""RMSNorm: y = x * rsqrt(mean(x^2) + eps) * gain, in 32-bit.

Reference: src/ops/kernels.hip:17-41; with the residual sum fused in,
:100-129. The residual stream is kept in 32-bit here (the reference keeps it
in half precision), so the sum is never rounded to the storage type.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..registry import register_part
from ..weights.source import TensorSpec
from .base import Norm, PendingRows, StepContext, WeightBinder


class RMSNorm(Norm):
    def __init__(self, prefix: str, size: int, eps: float):
        self.prefix = prefix
        self.size = size
        self.eps = eps
        self.gain: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {self.prefix + "weight": TensorSpec((self.size,), "gain")}

    def bind(self, w: WeightBinder) -> None:
        self.gain = w.float32(self.prefix + "weight")

    def forward(self, ctx: StepContext, residual, pending):
        out = ctx.empty((residual.shape[0], self.size))
        if isinstance(pending, PendingRows):
            ctx.ops.rmsnorm(residual, self.gain, self.eps, out, rows_sum=pending)
        else:
            ctx.ops.rmsnorm(residual, self.gain, self.eps, out, delta=pending)
        return out

    def forward_rows(self, ctx: StepContext, residual, rows, pending=None):
        out = ctx.empty((rows.shape[0], self.size))
        if isinstance(pending, PendingRows):
            ctx.ops.rmsnorm(residual, self.gain, self.eps, out, rows_sum=pending, rows=rows)
        else:
            ctx.ops.rmsnorm(residual, self.gain, self.eps, out, delta=pending, rows=rows)
        return out


register_part("norm", "rmsnorm", RMSNorm)
