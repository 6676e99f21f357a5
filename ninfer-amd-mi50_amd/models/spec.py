"""A model as data: its parts and the order they run in.

`blocks` are the model's layers; `plan` is the order they run in, one
`LayerCall` per run. The plan is data: it may name a layer twice (the layer's
weights run again, with a cache of their own unless told otherwise) or let a
call read the cache another call wrote (`cache_from`), in which case the call
writes no keys and values of its own.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional

import torch

from ..parts.base import Block, CallInfo, Norm, Part, StepContext, WeightBinder
from ..parts.embedding import LMHead, TokenEmbedding
from ..weights.source import TensorSpec


@dataclass(frozen=True)
class LayerCall:
    layer: int                       # index into ModelSpec.blocks
    cache_from: Optional[int] = None  # index of an earlier plan entry whose cache is read


class ModelSpec:
    def __init__(self, embedding: TokenEmbedding, blocks: List[Block], final_norm: Norm,
                 head: LMHead, plan: Optional[List[LayerCall]] = None,
                 vocab_size: Optional[int] = None, eos_token_ids=()):
        self.embedding = embedding
        self.blocks = blocks
        self.final_norm = final_norm
        self.head = head
        self.vocab_size = vocab_size if vocab_size is not None else head.vocab
        self.eos_token_ids = tuple(eos_token_ids)   # ids that end a generation by default
        self.plan: List[LayerCall] = []
        self.set_plan(plan if plan is not None else [LayerCall(i) for i in range(len(blocks))])

    def set_plan(self, plan: List[LayerCall]) -> None:
        """Replace the order the layers run in (before the model is bound to a
        cache); refuses entries that name no layer or read a cache that is not
        written earlier."""
        for i, call in enumerate(plan):
            if not 0 <= call.layer < len(self.blocks):
                raise ValueError(f"plan entry {i} names layer {call.layer}; the model has "
                                 f"{len(self.blocks)}")
            if call.cache_from is not None:
                if not 0 <= call.cache_from < i:
                    raise ValueError(f"plan entry {i} reads the cache of entry "
                                     f"{call.cache_from}, which does not run before it")
                if plan[call.cache_from].cache_from is not None:
                    raise ValueError(f"plan entry {i} reads the cache of entry "
                                     f"{call.cache_from}, which has no cache of its own")
        self.plan = list(plan)

    def parts(self) -> List[Part]:
        return [self.embedding, *self.blocks, self.final_norm, self.head]

    def max_positions(self) -> Optional[int]:
        """The longest request the parts allow (None: no part limits it)."""
        limits = [x for x in (p.least_max_positions() for p in self.parts()) if x is not None]
        return min(limits) if limits else None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        out: Dict[str, TensorSpec] = {}
        for p in self.parts():
            out.update(p.all_tensor_specs())
        return out

    def unused_tensor_specs(self) -> Dict[str, TensorSpec]:
        out: Dict[str, TensorSpec] = {}
        for p in self.parts():
            out.update(p.all_unused_tensor_specs())
        return out

    def bind(self, w: WeightBinder) -> None:
        for p in self.parts():
            p.bind_all(w)

    # ---- one step over the rows of `ctx` -----------------------------------
    def forward(self, ctx: StepContext, calls: List[CallInfo],
                logit_rows: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
        """Run all plan entries over the step's rows; logits [R, vocab] (32-bit)
        at `logit_rows`, or None when no logits are asked for."""
        residual = self.embedding.forward(ctx)
        pending = None
        for call, info in zip(self.plan, calls):
            pending = self.blocks[call.layer].forward(ctx, residual, pending, info)
        if logit_rows is None or logit_rows.numel() == 0:
            return None
        normed = self.final_norm.forward_rows(ctx, residual, logit_rows, pending)
        return self.head.forward(ctx, normed)
