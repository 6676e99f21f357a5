"""Dense SwiGLU feed-forward: (silu(x Wg^T) * (x Wu^T)) Wd^T, no biases.

Gate and up weights are stacked into one [2 I, hidden] matrix, rows [0, I)
gate and [I, 2I) up (reference src/models/model.hip:585-617); the activation
runs in the product's epilogue (the reference does so only for one row,
src/ops/gemv.hip:103-166, and otherwise in a kernel of its own,
src/ops/kernels.hip:131-140).
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..registry import register_part
from ..weights.source import TensorSpec
from .base import FeedForward, StepContext, WeightBinder


class SwiGLU(FeedForward):
    def __init__(self, prefix: str, hidden: int, inner: int, act: str = "silu", bias: bool = False):
        self.prefix = prefix
        self.hidden = hidden
        self.inner = inner
        self.act = act   # the gate's activation, by config.json's name: 'silu' | 'gelu_pytorch_tanh'
        self.bias = bias   # gate_proj.bias, up_proj.bias [inner] and down_proj.bias [hidden] are read
        self.w_gate_up: Optional[torch.Tensor] = None
        self.w_down: Optional[torch.Tensor] = None
        self.b_gate_up: Optional[torch.Tensor] = None
        self.b_down: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        p = self.prefix
        specs = {p + "gate_proj.weight": TensorSpec((self.inner, self.hidden)),
                 p + "up_proj.weight": TensorSpec((self.inner, self.hidden)),
                 p + "down_proj.weight": TensorSpec((self.hidden, self.inner))}
        if self.bias:
            specs[p + "gate_proj.bias"] = TensorSpec((self.inner,), "bias")
            specs[p + "up_proj.bias"] = TensorSpec((self.inner,), "bias")
            specs[p + "down_proj.bias"] = TensorSpec((self.hidden,), "bias")
        return specs

    def bind(self, w: WeightBinder) -> None:
        p = self.prefix
        self.w_gate_up = torch.empty((2 * self.inner, self.hidden), dtype=w.act_dtype,
                                     device=w.device)
        w.matrix_into(p + "gate_proj.weight", self.w_gate_up[:self.inner])
        w.matrix_into(p + "up_proj.weight", self.w_gate_up[self.inner:])
        self.w_down = w.matrix(p + "down_proj.weight")
        if self.bias:
            self.b_gate_up = torch.cat([w.float32(p + "gate_proj.bias"), w.float32(p + "up_proj.bias")])
            w.hold(p + "gate_proj.bias", self.b_gate_up[:self.inner])
            w.hold(p + "up_proj.bias", self.b_gate_up[self.inner:])
            self.b_down = w.float32(p + "down_proj.bias")

    def weight_bytes(self) -> int:
        """What one pass over the two weight matrices reads."""
        return 3 * self.inner * self.hidden * self.w_down.element_size()

    def gate_up(self, ctx: StepContext, x: torch.Tensor) -> torch.Tensor:
        h = ctx.empty((x.shape[0], self.inner))
        ctx.ops.swiglu_linear(x, self.w_gate_up, h, act=self.act, bias=self.b_gate_up)
        return h

    def down(self, ctx: StepContext, h: torch.Tensor) -> torch.Tensor:
        out = ctx.empty((h.shape[0], self.hidden))
        ctx.ops.linear(h, self.w_down, out, bias=self.b_down)
        return out

    def run(self, ctx: StepContext, x: torch.Tensor) -> torch.Tensor:
        return self.down(ctx, self.gate_up(ctx, x))

    def forward(self, ctx: StepContext, x, residual):
        return self.run(ctx, x)


register_part("feed_forward", "swiglu", SwiGLU)
