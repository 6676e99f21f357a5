"""What every part of a model is: its interface and the data a step hands it.

A model is put together from parts: a mixer (attention here), a feed-forward
(dense or experts), norms, a position encoding, and a block that arranges
them. A part has its sizes and constants as constructor parameters, names the
checkpoint tensors it needs, and runs on the rows of one step. No part knows
which model it is in: it sees its own parameters, a name prefix, and a
`StepContext`.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

import torch

from ..weights.source import TensorSpec


@dataclass(frozen=True)
class CacheNeed:
    """What a mixer needs of the paged cache for each token it has seen: keys
    and values of `kv_heads` heads of `head_dim`, all of them (window None) or
    only the last `window` positions."""
    kv_heads: int
    head_dim: int
    window: Optional[int] = None


@dataclass
class CacheView:
    """One cache instance as a step sees it: the layer's page pools
    [pages, kv_heads, page_size, head_dim] and the block table of the step's
    requests [S, max_pages] (int32, -1 where a page was given back)."""
    k_pool: torch.Tensor
    v_pool: torch.Tensor
    block_table: torch.Tensor
    page_size: int
    window: Optional[int]


@dataclass
class CallInfo:
    """How one entry of the layer plan runs: which cache it uses, whether it
    writes it (false when it reads another call's cache), and the slice of the
    per-request state that belongs to its mixer ([slots, floats], or None)."""
    cache: Optional[CacheView] = None
    writes_cache: bool = True
    state: Optional[torch.Tensor] = None


@dataclass
class StepContext:
    """The rows of one step and what parts need to run them.

    T rows of S requests; rows of one request are contiguous and in order.
    All index tensors are int32 on the device. `host` holds the same numbers as
    Python lists for sizing launches without a device round trip.
    """
    ops: Any
    act_dtype: torch.dtype
    device: torch.device
    T: int
    S: int
    tokens: torch.Tensor          # [T]
    positions: torch.Tensor       # [T] absolute position of each row in its request
    row_seq: torch.Tensor         # [T] index (within this step) of the row's request
    seq_slots: torch.Tensor       # [S] slot of each request (index into state)
    seq_row_start: torch.Tensor   # [S + 1] first row of each request, then T
    seq_qlen: torch.Tensor        # [S]
    seq_pos0: torch.Tensor        # [S] position of the request's first row
    max_qlen: int = 1
    max_kv_len: int = 1
    all_decode: bool = False
    single_rows: int = 0          # the first single_rows requests bring one row each (rows 0 ..)
    scratch: Dict[str, Any] = field(default_factory=dict)

    def empty(self, shape, dtype=None) -> torch.Tensor:
        return torch.empty(shape, dtype=dtype or self.act_dtype, device=self.device)


@dataclass
class PendingRows:
    """A weighted sum of rows that a part leaves to be added to the residual by
    whoever comes next (a norm's kernel adds it on the fly):
    sum_j weights[t, j] * y[t * k + j, :] + sigmoid(gate[t]) * shared[t, :].
    `shared` and `gate` may be None (no such term / factor 1). `gate` is a
    32-bit view [T] that may be strided."""
    y: torch.Tensor
    weights: torch.Tensor
    shared: Optional[torch.Tensor] = None
    gate: Optional[torch.Tensor] = None

    def add_to(self, ctx: "StepContext", residual: torch.Tensor) -> None:
        ctx.ops.moe_combine(residual, self.y, self.weights, self.shared, self.gate)


def settle(ctx: "StepContext", residual: torch.Tensor, pending) -> Optional[torch.Tensor]:
    """For parts that take only plain rows: a PendingRows is added into the
    residual now; a tensor (or None) is handed back unchanged."""
    if isinstance(pending, PendingRows):
        pending.add_to(ctx, residual)
        return None
    return pending


class WeightBinder:
    """Reads tensors by name from a weight source and places them on the
    device: matrices in the compute dtype, gains and biases in 32-bit."""

    def __init__(self, source: Any, device: torch.device, act_dtype: torch.dtype):
        self.source = source
        self.device = device
        self.act_dtype = act_dtype

    def matrix(self, name: str) -> torch.Tensor:
        return self.source.read(name).to(device=self.device, dtype=self.act_dtype).contiguous()

    def float32(self, name: str) -> torch.Tensor:
        return self.source.read(name).to(device=self.device, dtype=torch.float32).contiguous()

    def matrix_into(self, name: str, out: torch.Tensor) -> None:
        """Copy a matrix into a slice of a larger (fused or stacked) tensor."""
        out.copy_(self.source.read(name).to(device=self.device), non_blocking=False)


class Part:
    """Base of all parts. `prefix` is the part's checkpoint name prefix."""

    prefix: str = ""

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        """Full checkpoint names this part needs -> expected shape and role."""
        return {}

    def unused_tensor_specs(self) -> Dict[str, TensorSpec]:
        """Checkpoint names that may be there and that this part does not read
        (a copy of a tied table, a stored table of constants): present with the
        shape given they are passed over, absent they are not missed."""
        return {}

    def bind(self, w: WeightBinder) -> None:
        """Read this part's tensors (fusing or stacking them as its kernels
        want them)."""

    def children(self) -> List["Part"]:
        return []

    def all_tensor_specs(self) -> Dict[str, TensorSpec]:
        out = dict(self.tensor_specs())
        for c in self.children():
            out.update(c.all_tensor_specs())
        return out

    def all_unused_tensor_specs(self) -> Dict[str, TensorSpec]:
        out = dict(self.unused_tensor_specs())
        for c in self.children():
            out.update(c.all_unused_tensor_specs())
        return out

    def bind_all(self, w: WeightBinder) -> None:
        self.bind(w)
        for c in self.children():
            c.bind_all(w)


class Norm(Part):
    """y = norm(residual [+ pending]); the sum is kept in `residual` (32-bit).
    `pending` is rows [T, hidden], a PendingRows, or None (a norm that cannot
    add a PendingRows on the fly calls `settle` first)."""

    def forward(self, ctx: StepContext, residual: torch.Tensor,
                pending: Optional[torch.Tensor]) -> torch.Tensor:
        raise NotImplementedError

    def forward_rows(self, ctx: StepContext, residual: torch.Tensor, rows: torch.Tensor,
                     pending: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Norm of selected rows of residual [+ pending]; `residual` is left as
        it is."""
        raise NotImplementedError


class PositionEncoding(Part):
    """A position encoding applied to queries and keys inside a mixer."""

    rot_dim: int = 0

    def table(self) -> Optional[torch.Tensor]:
        raise NotImplementedError


class Mixer(Part):
    """Mixes information between the positions of a request.

    `cache_need()` says what it keeps per token in pages (None: nothing),
    `state_floats()` how many 32-bit numbers of fixed-size state it keeps per
    request (0: none). `forward` takes the normed rows [T, hidden] and returns
    rows [T, hidden] that the block adds to the residual.
    """

    def cache_need(self) -> Optional[CacheNeed]:
        return None

    def state_floats(self) -> int:
        return 0

    def forward(self, ctx: StepContext, x: torch.Tensor, residual: torch.Tensor,
                call: CallInfo) -> Optional[torch.Tensor]:
        raise NotImplementedError


class FeedForward(Part):
    """Row-wise transform. `forward` returns what is to be added to the
    residual: rows [T, hidden], a PendingRows, or None if it has already added
    its result to `residual` itself."""

    def forward(self, ctx: StepContext, x: torch.Tensor, residual: torch.Tensor
                ) -> Optional[torch.Tensor]:
        raise NotImplementedError


class Block(Part):
    """Arrangement of norms, mixer and feed-forward around the residual."""

    mixer: Mixer

    def forward(self, ctx: StepContext, residual: torch.Tensor,
                pending: Optional[torch.Tensor], call: CallInfo) -> Optional[torch.Tensor]:
        raise NotImplementedError
