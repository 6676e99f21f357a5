"""Sparse feed-forward: a router, routed experts, and an optional gated
shared expert.

Router (reference src/ops/moe.hip:65-82, there on the host with a sync per
layer): logits = x Wr^T in 32-bit, softmax over all experts, the k largest
(ties to the lower index), weights renormalised over the chosen only when
`renorm`. Routed experts (reference src/models/model.hip:352-433): each chosen
expert is a SwiGLU; rows are grouped by expert on the device (no host sync)
and run as one grouped product for gate/up and one for down. The shared
expert is a dense SwiGLU scaled per token by sigmoid(x w_gate^T). The result
sum_k w_k y_k + gamma s is accumulated into the 32-bit residual in a fixed
order (the reference scatter-adds half-precision rows, src/ops/moe.hip:22-31).
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..registry import register_part
from ..weights.source import TensorSpec
from .base import FeedForward, Part, StepContext, WeightBinder
from .mlp import SwiGLU


class SoftmaxTopKRouter(Part):
    def __init__(self, prefix: str, hidden: int, experts: int, top_k: int, renorm: bool):
        if top_k > experts:
            raise ValueError(f"top_k ({top_k}) exceeds the number of experts ({experts})")
        self.prefix = prefix
        self.hidden = hidden
        self.experts = experts
        self.top_k = top_k
        self.renorm = renorm
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {self.prefix + "weight": TensorSpec((self.experts, self.hidden))}

    def bind(self, w: WeightBinder) -> None:
        self.weight = w.matrix(self.prefix + "weight")

    def route(self, ctx: StepContext, x: torch.Tensor):
        t = x.shape[0]
        logits = ctx.empty((t, self.experts), torch.float32)
        ctx.ops.linear(x, self.weight, logits)
        ids = ctx.empty((t, self.top_k), torch.int32)
        wts = ctx.empty((t, self.top_k), torch.float32)
        ctx.ops.router_topk(logits, self.experts, self.top_k, self.renorm, ids, wts)
        return ids, wts


class RoutedExperts(Part):
    """E SwiGLU experts with stacked weights [E, 2I, hidden] and [E, hidden, I]
    built from the per-expert checkpoint tensors `experts.{e}.*_proj.weight`."""

    def __init__(self, prefix: str, hidden: int, inner: int, experts: int):
        self.prefix = prefix
        self.hidden = hidden
        self.inner = inner
        self.experts = experts
        self.w_gate_up: Optional[torch.Tensor] = None
        self.w_down: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs = {}
        for e in range(self.experts):
            p = f"{self.prefix}{e}."
            specs[p + "gate_proj.weight"] = TensorSpec((self.inner, self.hidden))
            specs[p + "up_proj.weight"] = TensorSpec((self.inner, self.hidden))
            specs[p + "down_proj.weight"] = TensorSpec((self.hidden, self.inner))
        return specs

    def bind(self, w: WeightBinder) -> None:
        i = self.inner
        self.w_gate_up = torch.empty((self.experts, 2 * i, self.hidden), dtype=w.act_dtype,
                                     device=w.device)
        self.w_down = torch.empty((self.experts, self.hidden, i), dtype=w.act_dtype,
                                  device=w.device)
        for e in range(self.experts):
            p = f"{self.prefix}{e}."
            w.matrix_into(p + "gate_proj.weight", self.w_gate_up[e, :i])
            w.matrix_into(p + "up_proj.weight", self.w_gate_up[e, i:])
            w.matrix_into(p + "down_proj.weight", self.w_down[e])

    def run(self, ctx: StepContext, x: torch.Tensor, ids: torch.Tensor) -> torch.Tensor:
        """Expert outputs [T*k, hidden], row t*k + j for the j-th choice of row t."""
        t, k = ids.shape
        offsets = ctx.empty((self.experts + 1,), torch.int32)
        order = ctx.empty((t * k,), torch.int32)
        ctx.ops.moe_align(ids, self.experts, offsets, order)
        h = ctx.empty((t * k, self.inner))
        ctx.ops.grouped_swiglu(x, self.w_gate_up, offsets, order, k, h)
        y = ctx.empty((t * k, self.hidden))
        ctx.ops.grouped_down(h, self.w_down, offsets, order, y)
        return y


class SparseMoE(FeedForward):
    def __init__(self, prefix: str, hidden: int, experts: int, top_k: int, inner: int,
                 renorm: bool, shared_inner: int = 0):
        self.prefix = prefix
        self.hidden = hidden
        self.router = SoftmaxTopKRouter(prefix + "gate.", hidden, experts, top_k, renorm)
        self.experts = RoutedExperts(prefix + "experts.", hidden, inner, experts)
        self.shared: Optional[SwiGLU] = None
        self.shared_gate: Optional[torch.Tensor] = None
        self.last_ids: Optional[torch.Tensor] = None   # routing of the last step (for statistics)
        if shared_inner > 0:
            self.shared = SwiGLU(prefix + "shared_expert.", hidden, shared_inner)

    def children(self) -> List[Part]:
        return [self.router, self.experts] + ([self.shared] if self.shared else [])

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        if self.shared is None:
            return {}
        return {self.prefix + "shared_expert_gate.weight": TensorSpec((1, self.hidden))}

    def bind(self, w: WeightBinder) -> None:
        if self.shared is not None:
            self.shared_gate = w.matrix(self.prefix + "shared_expert_gate.weight")

    def forward(self, ctx: StepContext, x, residual):
        ids, wts = self.router.route(ctx, x)
        self.last_ids = ids
        y = self.experts.run(ctx, x, ids)
        shared = gate = None
        if self.shared is not None:
            shared = self.shared.run(ctx, x)
            gate = ctx.empty((x.shape[0], 1), torch.float32)
            ctx.ops.linear(x, self.shared_gate, gate)
        ctx.ops.moe_combine(residual, y, wts, shared, gate)
        return None


register_part("feed_forward", "sparse_moe", SparseMoE)
