"""Pre-norm residual block: x += mixer(norm1(x)); x += feed_forward(norm2(x)).

Reference order: src/models/model.hip:206-444 (layer_start, layer_mid,
end_layer). A part's output is not added at once: it is handed on as
`pending` and summed into the 32-bit residual by the next norm's kernel (the
reference fuses the same sum with the post-attention norm only,
src/ops/kernels.hip:100-129).
"""
from __future__ import annotations

from typing import List, Optional

from ..registry import register_part
from .base import Block, CallInfo, FeedForward, Mixer, Norm, Part, StepContext


class PreNormBlock(Block):
    def __init__(self, mixer_norm: Norm, mixer: Mixer, ff_norm: Norm, feed_forward: FeedForward):
        self.mixer_norm = mixer_norm
        self.mixer = mixer
        self.ff_norm = ff_norm
        self.feed_forward = feed_forward

    def children(self) -> List[Part]:
        return [self.mixer_norm, self.mixer, self.ff_norm, self.feed_forward]

    def forward(self, ctx: StepContext, residual, pending, call: CallInfo):
        a = self.mixer_norm.forward(ctx, residual, pending)
        pending = self.mixer.forward(ctx, a, residual, call)
        m = self.ff_norm.forward(ctx, residual, pending)
        return self.feed_forward.forward(ctx, m, residual)


register_part("block", "pre_norm", PreNormBlock)
