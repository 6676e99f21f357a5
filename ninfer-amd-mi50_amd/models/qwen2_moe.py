"""Qwen2-MoE put together from parts, layer by layer from its configuration.

Per layer: RMSNorm -> attention (q/k/v bias unless `qkv_bias` is false, rotary, window on layers >=
max_window_layers when use_sliding_window) -> RMSNorm -> feed-forward, which
is sparse (router, routed experts, gated shared expert) or a dense SwiGLU of
`intermediate_size` according to `mlp_only_layers` and `decoder_sparse_step`.
Layer loop and tensor names: reference src/models/model.hip:509-583,
:1021-1025 (which builds every layer sparse and has no shared expert).
"""
from __future__ import annotations

from ..config.qwen2_moe import Qwen2MoeConfig
from ..parts.attention import Attention
from ..parts.block import PreNormBlock
from ..parts.embedding import LMHead, TokenEmbedding
from ..parts.mlp import SwiGLU
from ..parts.moe import SparseMoE
from ..parts.norm import RMSNorm
from ..parts.rotary import Rotary
from ..registry import register_architecture
from .spec import ModelSpec


def build_qwen2_moe(cfg: Qwen2MoeConfig) -> ModelSpec:
    h = cfg.hidden_size
    rotary = Rotary(cfg.head_dim, cfg.rope_theta)
    embedding = TokenEmbedding("model.embed_tokens.", cfg.vocab_size, h)
    blocks = []
    for l in range(cfg.num_hidden_layers):
        p = f"model.layers.{l}."
        mixer = Attention(p + "self_attn.", h, cfg.num_attention_heads, cfg.num_key_value_heads,
                          cfg.head_dim, rotary, qkv_bias=cfg.qkv_bias, window=cfg.layer_window(l))
        if cfg.layer_is_sparse(l):
            ff = SparseMoE(p + "mlp.", h, cfg.num_experts, cfg.num_experts_per_tok,
                           cfg.moe_intermediate_size, cfg.norm_topk_prob,
                           cfg.shared_expert_intermediate_size)
        else:
            ff = SwiGLU(p + "mlp.", h, cfg.intermediate_size)
        blocks.append(PreNormBlock(RMSNorm(p + "input_layernorm.", h, cfg.rms_norm_eps), mixer,
                                   RMSNorm(p + "post_attention_layernorm.", h, cfg.rms_norm_eps),
                                   ff))
    final_norm = RMSNorm("model.norm.", h, cfg.rms_norm_eps)
    head = LMHead("lm_head.", cfg.vocab_size, h,
                  tied_to=embedding if cfg.tie_word_embeddings else None)
    return ModelSpec(embedding, blocks, final_norm, head, eos_token_id=cfg.eos_token_id)


register_architecture("Qwen2MoeForCausalLM", Qwen2MoeConfig.from_dict, build_qwen2_moe)
