"""Token embedding and the logits head.

Embedding: x[t] = table[token[t]] (reference src/ops/kernels.hip:150-159),
written straight into the 32-bit residual. Head: logits = n W^T in 32-bit for
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
    def __init__(self, prefix: str, vocab: int, hidden: int):
        self.prefix = prefix
        self.vocab = vocab
        self.hidden = hidden
        self.table: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {self.prefix + "weight": TensorSpec((self.vocab, self.hidden))}

    def bind(self, w: WeightBinder) -> None:
        self.table = w.matrix(self.prefix + "weight")

    def forward(self, ctx: StepContext) -> torch.Tensor:
        residual = ctx.empty((ctx.T, self.hidden), torch.float32)
        ctx.ops.embed(ctx.tokens, self.table, residual)
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
