"""Token embedding and the logits head.

Embedding: x[t] = table[token[t]] (reference src/ops/kernels.hip:150-159),
written straight into the 32-bit residual; with `positions` > 0 a table of that many learned
absolute positions (`position_prefix + "weight"`) is gathered by the rows' positions and added
in the same kernel (no counterpart in the reference: its models rotate). Head: logits = n W^T in 32-bit for
the asked rows only (reference src/models/model.hip:735-752); with tied
embeddings the head is the embedding table itself, not a copy (the reference
loads a second copy, :496-500).
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..weights.source import TensorSpec
from .base import Part, StepContext, WeightBinder


class TokenEmbedding(Part):
    def __init__(self, prefix: str, vocab: int, hidden: int, positions: int = 0,
                 position_prefix: Optional[str] = None):
        self.prefix = prefix
        self.vocab = vocab
        self.hidden = hidden
        self.positions = positions   # rows of the table of learned positions (0: none)
        self.position_prefix = position_prefix
        if positions and not position_prefix:
            raise ValueError("learned positions need the name prefix of their table")
        self.table: Optional[torch.Tensor] = None
        self.position_table: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs = {self.prefix + "weight": TensorSpec((self.vocab, self.hidden))}
        if self.positions:
            specs[self.position_prefix + "weight"] = TensorSpec((self.positions, self.hidden))
        return specs

    def bind(self, w: WeightBinder) -> None:
        self.table = w.matrix(self.prefix + "weight")
        if self.positions:
            self.position_table = w.matrix(self.position_prefix + "weight")

    def max_positions(self) -> Optional[int]:
        return self.positions or None

    def forward(self, ctx: StepContext) -> torch.Tensor:
        residual = ctx.empty((ctx.T, self.hidden), torch.float32)
        ctx.ops.embed(ctx.tokens, self.table, residual, positions=ctx.positions,
                      pos_table=self.position_table)
        return residual


class LMHead(Part):
    def __init__(self, prefix: str, vocab: int, hidden: int,
                 tied_to: Optional[TokenEmbedding] = None):
        self.prefix = prefix
        self.vocab = vocab
        self.hidden = hidden
        self.tied_to = tied_to
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        if self.tied_to is not None:
            return {}
        return {self.prefix + "weight": TensorSpec((self.vocab, self.hidden))}

    def unused_tensor_specs(self) -> Dict[str, TensorSpec]:
        # a checkpoint of a tied model may still carry the head: a copy of the table
        if self.tied_to is not None:
            return {self.prefix + "weight": TensorSpec((self.vocab, self.hidden))}
        return {}

    def bind(self, w: WeightBinder) -> None:
        if self.tied_to is None:
            self.weight = w.matrix(self.prefix + "weight")

    def forward(self, ctx: StepContext, normed_rows: torch.Tensor) -> torch.Tensor:
        weight = self.tied_to.table if self.tied_to is not None else self.weight
        logits = ctx.empty((normed_rows.shape[0], self.vocab), torch.float32)
        ctx.ops.linear(normed_rows, weight, logits)
        return logits
