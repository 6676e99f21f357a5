"""Qwen2-MoE put together from parts, layer by layer from its configuration.

Per layer: RMSNorm -> attention (q/k/v bias unless `qkv_bias` is false, rotary, window on layers >=
max_window_layers when use_sliding_window) -> RMSNorm -> feed-forward, which
is sparse (router, routed experts, gated shared expert) or a dense SwiGLU of
`intermediate_size` according to `mlp_only_layers` and `decoder_sparse_step`.
Layer loop and tensor names: reference src/models/model.hip:509-583,
:1021-1025 (which builds every layer sparse and has no shared expert).
"""
from __future__ import annotations

from .. import parts  # noqa: F401  (registers the part factories by kind and name)
from ..config.qwen2_moe import Qwen2MoeConfig
from ..parts.embedding import LMHead, TokenEmbedding
from ..registry import make_part, register_architecture
from .spec import ModelSpec


def build_qwen2_moe(cfg: Qwen2MoeConfig) -> ModelSpec:
    """Every part of a layer is made by kind and name through the part registry, so a
    builder of another architecture chooses other names (its own, registered from outside
    the package, or these) layer by layer in the same way."""
    h = cfg.hidden_size
    rotary = make_part("position", "rotary", rot_dim=cfg.head_dim, theta=cfg.rope_theta)
    embedding = TokenEmbedding("model.embed_tokens.", cfg.vocab_size, h)
    blocks = []
    for l in range(cfg.num_hidden_layers):
        p = f"model.layers.{l}."
        mixer = make_part("mixer", "attention", prefix=p + "self_attn.", hidden=h,
                          heads=cfg.num_attention_heads, kv_heads=cfg.num_key_value_heads,
                          head_dim=cfg.head_dim, position=rotary, qkv_bias=cfg.qkv_bias,
                          window=cfg.layer_window(l))
        if cfg.layer_is_sparse(l):
            ff = make_part("feed_forward", "sparse_moe", prefix=p + "mlp.", hidden=h,
                           experts=cfg.num_experts, top_k=cfg.num_experts_per_tok,
                           inner=cfg.moe_intermediate_size, renorm=cfg.norm_topk_prob,
                           shared_inner=cfg.shared_expert_intermediate_size,
                           act=cfg.hidden_act)
        else:
            ff = make_part("feed_forward", "swiglu", prefix=p + "mlp.", hidden=h,
                           inner=cfg.intermediate_size, act=cfg.hidden_act)
        norm = lambda name: make_part("norm", "rmsnorm", prefix=p + name, size=h,
                                      eps=cfg.rms_norm_eps)
        blocks.append(make_part("block", "pre_norm", mixer_norm=norm("input_layernorm."),
                                mixer=mixer, ff_norm=norm("post_attention_layernorm."),
                                feed_forward=ff))
    final_norm = make_part("norm", "rmsnorm", prefix="model.norm.", size=h, eps=cfg.rms_norm_eps)
    head = LMHead("lm_head.", cfg.vocab_size, h,
                  tied_to=embedding if cfg.tie_word_embeddings else None)
    return ModelSpec(embedding, blocks, final_norm, head, eos_token_ids=cfg.eos_token_ids)


register_architecture("Qwen2MoeForCausalLM", Qwen2MoeConfig.from_dict, build_qwen2_moe)
