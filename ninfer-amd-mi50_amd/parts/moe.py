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
from .base import FeedForward, Part, PendingRows, StepContext, WeightBinder
from .mlp import SwiGLU


class TopKRouter(Part):
    """logits = x Wr^T (32-bit); scores s = softmax over all experts, or sigmoid of each
    logit (`score`); the `top_k` experts with the largest s (+ a per-expert bias of the
    checkpoint, `prefix + "choice_bias"`, when `choice_bias`: it decides the choice only)
    are chosen, ties to the lower index; their weights are their scores, divided by their
    sum when `renorm`, times `scale`. Softmax without bias and scale 1 is this
    architecture's router (reference src/ops/moe.hip:65-82, which always renormalises)."""

    def __init__(self, prefix: str, hidden: int, experts: int, top_k: int, renorm: bool,
                 score: str = "softmax", scale: float = 1.0, choice_bias: bool = False,
                 n_group: int = 0, topk_group: int = 0):
        if top_k > experts:
            raise ValueError(f"top_k ({top_k}) exceeds the number of experts ({experts})")
        if score not in ("softmax", "sigmoid"):
            raise ValueError(f"score must be 'softmax' or 'sigmoid', got {score!r}")
        self.prefix = prefix
        self.hidden = hidden
        self.experts = experts
        self.top_k = top_k
        self.renorm = renorm
        self.score = score
        self.scale = float(scale)
        self.has_choice_bias = choice_bias
        # a group-limited choice: only the experts of the topk_group groups (of experts /
        # n_group neighbours each) whose best score (+ bias) is largest are candidates
        self.n_group, self.topk_group = int(n_group), int(topk_group)
        if self.n_group > 1 and (experts % self.n_group or not 1 <= self.topk_group <= self.n_group
                                 or self.topk_group * (experts // self.n_group) < top_k):
            raise ValueError(f"{self.n_group} groups of which {self.topk_group} are open do not fit "
                             f"{experts} experts and top_k {top_k}")
        self.weight: Optional[torch.Tensor] = None
        self.choice_bias: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs = {self.prefix + "weight": TensorSpec((self.experts, self.hidden))}
        if self.has_choice_bias:
            specs[self.prefix + "choice_bias"] = TensorSpec((self.experts,), role="bias")
        return specs

    def bind(self, w: WeightBinder) -> None:
        self.weight = w.matrix(self.prefix + "weight")
        if self.has_choice_bias:
            self.choice_bias = w.float32(self.prefix + "choice_bias")

    def logits(self, ctx: StepContext, x: torch.Tensor) -> torch.Tensor:
        out = ctx.empty((x.shape[0], self.experts), torch.float32)
        ctx.ops.linear(x, self.weight, out)
        return out

    def route(self, ctx: StepContext, logits: torch.Tensor) -> "Routing":
        """Choose experts from router logits [T, >= experts] (more columns are
        ignored) and group the routed rows by expert, all on the device."""
        t, k, e = logits.shape[0], self.top_k, self.experts
        n = t * k
        r = Routing(ids=ctx.empty((t, k), torch.int32), weights=ctx.empty((t, k), torch.float32),
                    offsets=ctx.empty((e + 1,), torch.int32), order=ctx.empty((n,), torch.int32),
                    tiles16=ctx.empty((min(n, n // 16 + e), 4), torch.int32),
                    tiles_big=ctx.empty((n // Routing.BIG_ROWS + e, 4), torch.int32),
                    tile_counts=ctx.empty((2,), torch.int32))
        ctx.ops.moe_route(logits, e, k, self.renorm, r, score=self.score,
                          choice_bias=self.choice_bias, scale=self.scale, n_group=self.n_group,
                          topk_group=self.topk_group)
        return r


SoftmaxTopKRouter = TopKRouter   # the default parameters: this architecture's router


class Routing:
    """What routing leaves on the device: chosen experts and weights per row,
    the (row, choice) indices grouped by expert (`order`, `offsets`), and the
    lists of 16-row and of tall (256-row) tiles the grouped products walk:
    `tiles16` [min(n, n // 16 + experts), 4], `tiles_big` [n // 256 + experts, 4]
    and `tile_counts` [2] for n routed rows, or all three None."""

    BIG_ROWS = 256   # rows of a tall tile: one height serves every count of rows per expert

    def __init__(self, ids, weights, offsets, order, tiles16=None, tiles_big=None,
                 tile_counts=None):
        self.ids, self.weights, self.offsets, self.order = ids, weights, offsets, order
        self.tiles16, self.tiles_big, self.tile_counts = tiles16, tiles_big, tile_counts
        self.parts = None   # scratch of the routing of many rows (made by the kernel library's call)


class RoutedExperts(Part):
    """E SwiGLU experts with stacked weights [E, 2I, hidden] and [E, hidden, I]
    built from the per-expert checkpoint tensors `experts.{e}.*_proj.weight`."""

    def __init__(self, prefix: str, hidden: int, inner: int, experts: int, act: str = "silu"):
        self.prefix = prefix
        self.hidden = hidden
        self.inner = inner
        self.experts = experts
        self.act = act
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

    def gate_up(self, ctx: StepContext, x: torch.Tensor, routing: "Routing") -> torch.Tensor:
        """Activations [T*k, inner] in sorted order (row r belongs to the expert that
        owns sorted position r)."""
        t, k = routing.ids.shape
        h = ctx.empty((t * k, self.inner))
        ctx.ops.grouped_swiglu(x, self.w_gate_up, routing.offsets, routing.order, k, h,
                               tiles=routing, act=self.act)
        return h

    def down(self, ctx: StepContext, h: torch.Tensor, routing: "Routing") -> torch.Tensor:
        """Expert outputs [T*k, hidden], row t*k + j for the j-th choice of row t."""
        y = ctx.empty((h.shape[0], self.hidden))
        ctx.ops.grouped_down(h, self.w_down, routing.offsets, routing.order, y, tiles=routing)
        return y

    def run(self, ctx: StepContext, x: torch.Tensor, routing: "Routing") -> torch.Tensor:
        return self.down(ctx, self.gate_up(ctx, x, routing), routing)


class SparseMoE(FeedForward):
    def __init__(self, prefix: str, hidden: int, experts: int, top_k: int, inner: int,
                 renorm: bool, shared_inner: int = 0, act: str = "silu"):
        self.prefix = prefix
        self.hidden = hidden
        self.router = SoftmaxTopKRouter(prefix + "gate.", hidden, experts, top_k, renorm)
        self.experts = RoutedExperts(prefix + "experts.", hidden, inner, experts, act)
        self.shared: Optional[SwiGLU] = None
        self.shared_gate: Optional[torch.Tensor] = None
        self.last_ids: Optional[torch.Tensor] = None   # routing of the last step (for statistics)
        if shared_inner > 0:
            self.shared = SwiGLU(prefix + "shared_expert.", hidden, shared_inner, act)

    def children(self) -> List[Part]:
        return [self.router, self.experts] + ([self.shared] if self.shared else [])

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        if self.shared is None:
            return {}
        return {self.prefix + "shared_expert_gate.weight": TensorSpec((1, self.hidden))}

    def bind(self, w: WeightBinder) -> None:
        if self.shared is not None:
            self.shared_gate = w.matrix(self.prefix + "shared_expert_gate.weight")

    def bind_all(self, w: WeightBinder) -> None:
        super().bind_all(w)
        if self.shared is not None:
            # one product gives the router logits and the shared expert's gate logit
            e = self.router.experts
            self.router_and_gate = torch.cat([self.router.weight, self.shared_gate])
            self.router.weight = self.router_and_gate[:e]
            self.shared_gate = self.router_and_gate[e:]
            w.hold(self.router.prefix + "weight", self.router.weight)
            w.hold(self.prefix + "shared_expert_gate.weight", self.shared_gate)

    def forward(self, ctx: StepContext, x, residual):
        if self.shared is None:
            with ctx.ops.together():   # for few rows the logits' block routes the rows itself
                routing = self.router.route(ctx, self.router.logits(ctx, x))
            self.last_ids = routing.ids
            return PendingRows(self.experts.run(ctx, x, routing), routing.weights)
        # The shared expert's two products wait for nothing the routed path makes. Many rows:
        # they run on a stream of their own beside the routed path, whose kernels leave part
        # of the device empty in their last round of blocks.
        logits = ctx.empty((x.shape[0], self.router.experts + 1), torch.float32)
        if ctx.ops.wants_beside(x.shape[0], self.shared.weight_bytes()):
            # routing first: its short kernels would crawl beside the shared expert's long ones
            ctx.ops.linear(x, self.router_and_gate, logits)
            routing = self.router.route(ctx, logits)
            self.last_ids = routing.ids
            with ctx.ops.beside():
                shared = self.shared.down(ctx, self.shared.gate_up(ctx, x))
            y = self.experts.run(ctx, x, routing)
            ctx.ops.join()
            return PendingRows(y, routing.weights, shared, logits[:, self.router.experts])
        # Few rows: each goes together with the routed path's product of the same stage.
        # The routing goes with them: for a handful of rows the block that computes the logits
        # routes the rows itself.
        with ctx.ops.together():
            ctx.ops.linear(x, self.router_and_gate, logits)
            h_shared = self.shared.gate_up(ctx, x)
            routing = self.router.route(ctx, logits)
        gate = logits[:, self.router.experts]
        self.last_ids = routing.ids
        h = self.experts.gate_up(ctx, x, routing)
        with ctx.ops.together():
            y = self.experts.down(ctx, h, routing)
            shared = self.shared.down(ctx, h_shared)
        # not added here: the next norm's kernel adds it to the residual on the fly
        return PendingRows(y, routing.weights, shared, gate)


register_part("feed_forward", "sparse_moe", SparseMoE)
