"""Grouped-query attention over the paged cache.

q, k, v = x W^T (+ b) as one fused product over the stacked weight
[(Hq + 2 Hkv) D, hidden] (the reference fuses the same way,
src/models/model.hip:529-558, but has no bias); q and k are rotated, k and v
are written into the request's pages, and every row attends to the keys of
its request at positions <= its own (reference src/ops/attention.hip:216),
within `window` positions if the layer has one. Query head h reads kv head
h // (Hq / Hkv) (src/ops/attention.hip:27-28); scale 1/sqrt(D)
(src/models/model.hip:285). The output projection has no bias.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence

import torch

from ..registry import register_part
from ..weights.source import TensorSpec
from .base import CacheNeed, CallInfo, Mixer, Part, PositionEncoding, StepContext, WeightBinder


class Attention(Mixer):
    def __init__(self, prefix: str, hidden: int, heads: int, kv_heads: int, head_dim: int,
                 position: PositionEncoding, qkv_bias: bool = True,
                 window: Optional[int] = None, scale: Optional[float] = None,
                 score_slopes: Optional[Sequence[float]] = None,
                 qk_norm_eps: Optional[float] = None, page_size: Optional[int] = None):
        """`score_slopes` [heads]: a distance-based position bias, slope * (key's position -
        query's position) added to head h's scaled scores before the softmax (None: none).
        It is a parameter of the attention kernels, beside or instead of the rotation that
        `position` describes. `qk_norm_eps`: every query and key head is normed over its dims
        (x rsqrt(mean(x^2) + eps) gain, gains `q_norm.weight` and `k_norm.weight` [head_dim] of the
        checkpoint) after the bias and before it turns; None: no such norm. `page_size`: tokens
        in a page of this layer's keys and values (None: the engine's)."""
        if heads % kv_heads:
            raise ValueError(f"heads ({heads}) must be a multiple of kv_heads ({kv_heads})")
        if score_slopes is not None and len(score_slopes) != heads:
            raise ValueError(f"score_slopes has {len(score_slopes)} entries for {heads} heads")
        self.prefix = prefix
        self.hidden = hidden
        self.heads = heads
        self.kv_heads = kv_heads
        self.head_dim = head_dim
        self.position = position
        self.qkv_bias = qkv_bias
        self.window = window
        self.scale = scale if scale is not None else 1.0 / math.sqrt(head_dim)
        self.score_slopes = None if score_slopes is None else [float(x) for x in score_slopes]
        self.slopes: Optional[torch.Tensor] = None   # the same on the device (32-bit)
        self.qk_norm_eps = qk_norm_eps
        self.page_size = page_size
        self.q_norm: Optional[torch.Tensor] = None
        self.k_norm: Optional[torch.Tensor] = None
        self.w_qkv: Optional[torch.Tensor] = None
        self.b_qkv: Optional[torch.Tensor] = None
        self.w_o: Optional[torch.Tensor] = None

    @property
    def qkv_width(self) -> int:
        return (self.heads + 2 * self.kv_heads) * self.head_dim

    def cache_need(self) -> Optional[CacheNeed]:
        return CacheNeed.keys_values(self.kv_heads, self.head_dim, self.window, self.page_size)

    def children(self) -> List[Part]:
        return [self.position]

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        p, d = self.prefix, self.head_dim
        specs = {
            p + "q_proj.weight": TensorSpec((self.heads * d, self.hidden)),
            p + "k_proj.weight": TensorSpec((self.kv_heads * d, self.hidden)),
            p + "v_proj.weight": TensorSpec((self.kv_heads * d, self.hidden)),
            p + "o_proj.weight": TensorSpec((self.hidden, self.heads * d)),
        }
        if self.qkv_bias:
            specs[p + "q_proj.bias"] = TensorSpec((self.heads * d,), "bias")
            specs[p + "k_proj.bias"] = TensorSpec((self.kv_heads * d,), "bias")
            specs[p + "v_proj.bias"] = TensorSpec((self.kv_heads * d,), "bias")
        if self.qk_norm_eps is not None:
            specs[p + "q_norm.weight"] = TensorSpec((d,), "gain")
            specs[p + "k_norm.weight"] = TensorSpec((d,), "gain")
        return specs

    def unused_tensor_specs(self) -> Dict[str, TensorSpec]:
        # older checkpoints store the rotation's frequency table, which is computed here
        if self.position.rot_dim > 0:
            return {self.prefix + "rotary_emb.inv_freq": TensorSpec((self.position.rot_dim // 2,))}
        return {}

    def bind(self, w: WeightBinder) -> None:
        p, d = self.prefix, self.head_dim
        nq, nk = self.heads * d, self.kv_heads * d
        if self.score_slopes is not None:
            self.slopes = torch.tensor(self.score_slopes, dtype=torch.float32, device=w.device)
        if self.qk_norm_eps is not None:
            self.q_norm = w.float32(p + "q_norm.weight")
            self.k_norm = w.float32(p + "k_norm.weight")
        self.w_qkv = torch.empty((self.qkv_width, self.hidden), dtype=w.act_dtype, device=w.device)
        w.matrix_into(p + "q_proj.weight", self.w_qkv[:nq])
        w.matrix_into(p + "k_proj.weight", self.w_qkv[nq:nq + nk])
        w.matrix_into(p + "v_proj.weight", self.w_qkv[nq + nk:])
        if self.qkv_bias:
            self.b_qkv = torch.cat([w.float32(p + "q_proj.bias"), w.float32(p + "k_proj.bias"),
                                    w.float32(p + "v_proj.bias")])
            w.hold(p + "q_proj.bias", self.b_qkv[:nq])
            w.hold(p + "k_proj.bias", self.b_qkv[nq:nq + nk])
            w.hold(p + "v_proj.bias", self.b_qkv[nq + nk:])
        self.w_o = w.matrix(p + "o_proj.weight")

    def forward(self, ctx: StepContext, x, residual, call: CallInfo):
        ops = ctx.ops
        cache = call.cache
        qkv = ctx.empty((ctx.T, self.qkv_width))
        # the product, then bias, rotation of q and k, and the write of k, v into pages
        ops.qkv_rope(x, self.w_qkv, self.b_qkv, qkv, ctx.positions, ctx.row_seq,
                     self.position.table(), self.position.rot_dim, self.heads, self.kv_heads,
                     self.head_dim, cache["k"], cache["v"], cache.block_table,
                     cache.page_size, write_kv=call.writes_cache,
                     interleaved=self.position.pairing == "interleaved",
                     q_norm=self.q_norm, k_norm=self.k_norm, norm_eps=self.qk_norm_eps or 0.0)
        attn = ctx.empty((ctx.T, self.heads * self.head_dim))
        ops.paged_attention(qkv, cache["k"], cache["v"], cache.block_table, ctx,
                            self.heads, self.kv_heads, self.head_dim,
                            cache.page_size, self.window, self.scale, attn, slopes=self.slopes)
        out = ctx.empty((ctx.T, self.hidden))
        ops.linear(attn, self.w_o, out)
        return out


register_part("mixer", "attention", Attention)
