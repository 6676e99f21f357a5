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
from typing import Any, Dict, List, Optional, Tuple

import torch

from ..weights.source import TensorSpec


@dataclass(frozen=True)
class PoolSpec:
    """One paged pool of a mixer: what it keeps per token under `name`.

    The pool's tensor is [pages, *outer, page_size, *inner]: `outer` are the
    dimensions a page is split by before its token slots (heads, for keys and
    values), `inner` what one token holds in one of them (a head's numbers).
    `dtype` None means the engine's activation dtype; 'float32' or 'bfloat16'
    fix it."""
    name: str
    outer: Tuple[int, ...]
    inner: Tuple[int, ...]
    dtype: Optional[str] = None

    def elements_per_token(self) -> int:
        n = 1
        for d in self.outer + self.inner:
            n *= d
        return n


@dataclass(frozen=True)
class CacheNeed:
    """What a mixer needs of the paged cache for each token it has seen: any
    number of named pools, each with a per-token shape and dtype of its own,
    for all positions (window None) or only the last `window` of them, in pages
    of `page_size` tokens (None: the engine's). Mixers with the same window and
    page size share page numbers and block tables; each has pools of its own."""
    pools: Tuple[PoolSpec, ...]
    window: Optional[int] = None
    page_size: Optional[int] = None

    @staticmethod
    def keys_values(kv_heads: int, head_dim: int, window: Optional[int] = None,
                    page_size: Optional[int] = None) -> "CacheNeed":
        """Keys and values of `kv_heads` heads of `head_dim`: pools 'k' and 'v',
        each [pages, kv_heads, page_size, head_dim]."""
        return CacheNeed((PoolSpec("k", (kv_heads,), (head_dim,)),
                          PoolSpec("v", (kv_heads,), (head_dim,))), window, page_size)


@dataclass
class CacheView:
    """One cache instance as a step sees it: the mixer's pools by name (each
    [pages, *outer, page_size, *inner]) and the block table of the step's
    requests [S, max_pages] (int32, -1 where a page was given back)."""
    pools: Dict[str, torch.Tensor]
    block_table: torch.Tensor
    page_size: int
    window: Optional[int]

    def __getitem__(self, name: str) -> torch.Tensor:
        return self.pools[name]


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
    device: matrices in the compute dtype, gains and biases in 32-bit. It keeps
    a record name -> the device tensor (or the slice of a fused or stacked one)
    that now holds that checkpoint tensor, so that what the engine holds can be
    read back by checkpoint name."""

    def __init__(self, source: Any, device: torch.device, act_dtype: torch.dtype):
        self.source = source
        self.device = device
        self.act_dtype = act_dtype
        self.held: Dict[str, torch.Tensor] = {}

    def hold(self, name: str, where: torch.Tensor) -> None:
        """Record (or correct, after a part has moved it) where a tensor lives."""
        self.held[name] = where

    def matrix(self, name: str) -> torch.Tensor:
        t = self.source.read(name).to(device=self.device, dtype=self.act_dtype).contiguous()
        self.held[name] = t
        return t

    def float32(self, name: str) -> torch.Tensor:
        t = self.source.read(name).to(device=self.device, dtype=torch.float32).contiguous()
        self.held[name] = t
        return t

    def matrix_into(self, name: str, out: torch.Tensor) -> None:
        """Copy a matrix into a slice of a larger (fused or stacked) tensor."""
        out.copy_(self.source.read(name).to(device=self.device), non_blocking=False)
        self.held[name] = out


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

    def max_positions(self) -> Optional[int]:
        """The most positions a request may have because of this part (a table of learned
        positions has so many rows), or None: no limit of its own. The engine refuses a
        `max_context` beyond the least of its parts' limits."""
        return None

    def least_max_positions(self) -> Optional[int]:
        limits = [self.max_positions()] + [c.least_max_positions() for c in self.children()]
        limits = [x for x in limits if x is not None]
        return min(limits) if limits else None

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
    """A position encoding applied to queries and keys inside a mixer: a
    rotation of the first `rot_dim` dims of every head, pair i by the angle
    pos * table()[i]. `pairing` says which dims form pair i: 'half' pairs
    (i, i + rot_dim / 2), 'interleaved' the neighbours (2i, 2i + 1). The table
    holds any frequencies (scaled per dimension or not); rot_dim 0 is no
    rotation."""

    rot_dim: int = 0
    pairing: str = "half"

    def table(self) -> Optional[torch.Tensor]:
        raise NotImplementedError


class Mixer(Part):
    """Mixes information between the positions of a request.

    `cache_need()` says what it keeps per token in pages (None: nothing; else
    named pools, each with its own per-token shape and dtype),
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
