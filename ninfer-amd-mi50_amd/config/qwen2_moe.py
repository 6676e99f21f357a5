"""Typed configuration of Qwen2-MoE (`Qwen2MoeForCausalLM`, model_type
`qwen2_moe`), read from the architecture's own config.json keys.

Keys and defaults the reference reads: src/models/config.cpp:12-43
(`num_key_value_heads` defaults to the head count :21-23, `head_dim` to
hidden/heads :25-27, `rope_theta` to 1e6 :29-30, `tie_word_embeddings` to
false :31-32). The keys it does not read (shared expert size, `norm_topk_prob`,
`decoder_sparse_step`, `mlp_only_layers`, the sliding-window keys, `qkv_bias`)
are read here because the architecture has them.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Tuple

from .base import ConfigError, KeyReader


@dataclass(frozen=True)
class Qwen2MoeConfig:
    vocab_size: int
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    rms_norm_eps: float
    rope_theta: float
    tie_word_embeddings: bool
    num_experts: int
    num_experts_per_tok: int
    moe_intermediate_size: int
    shared_expert_intermediate_size: int
    norm_topk_prob: bool
    decoder_sparse_step: int
    mlp_only_layers: List[int] = field(default_factory=list)
    use_sliding_window: bool = False
    sliding_window: Optional[int] = None
    max_window_layers: int = 0
    qkv_bias: bool = True
    hidden_act: str = "silu"   # the gate's activation in every feed-forward: 'silu' | 'gelu_pytorch_tanh'
    eos_token_ids: Tuple[int, ...] = ()   # every id that ends a generation (the key may hold one or a list)
    architecture: str = "Qwen2MoeForCausalLM"

    @property
    def eos_token_id(self) -> Optional[int]:
        return self.eos_token_ids[0] if self.eos_token_ids else None

    # ---- derived, layer by layer -------------------------------------
    def layer_is_sparse(self, layer: int) -> bool:
        """Experts on layer l iff l is not in mlp_only_layers, there are
        experts, and (l + 1) is a multiple of decoder_sparse_step."""
        return (layer not in self.mlp_only_layers and self.num_experts > 0
                and (layer + 1) % self.decoder_sparse_step == 0)

    def layer_window(self, layer: int) -> Optional[int]:
        """Window of layer l: `sliding_window` for l >= max_window_layers when
        use_sliding_window, else none."""
        if self.use_sliding_window and layer >= self.max_window_layers:
            return self.sliding_window
        return None

    @staticmethod
    def from_dict(raw: Dict[str, Any]) -> "Qwen2MoeConfig":
        r = KeyReader(raw)
        mt = r.opt_str("model_type", "qwen2_moe")
        if mt != "qwen2_moe":
            raise ConfigError(f"config.json: key 'model_type' must be 'qwen2_moe', got {mt!r}")
        vocab = r.need_int("vocab_size", 1)
        hidden = r.need_int("hidden_size", 1)
        layers = r.need_int("num_hidden_layers", 1)
        heads = r.need_int("num_attention_heads", 1)
        kv_heads = r.opt_int("num_key_value_heads", heads, 1)
        inter = r.need_int("intermediate_size", 1)
        head_dim = r.opt_int("head_dim", None, 1)
        if head_dim is None:
            if hidden % heads:
                raise ConfigError("config.json: 'hidden_size' is not a multiple of "
                                  "'num_attention_heads' and 'head_dim' is not given")
            head_dim = hidden // heads
        if heads % kv_heads:
            raise ConfigError(f"config.json: 'num_attention_heads' ({heads}) must be a "
                              f"multiple of 'num_key_value_heads' ({kv_heads})")
        if head_dim % 2:
            raise ConfigError(f"config.json: 'head_dim' must be even, got {head_dim}")
        eps = r.need_float("rms_norm_eps")
        if not eps > 0:
            raise ConfigError(f"config.json: key 'rms_norm_eps' must be > 0, got {eps}")
        # the rotation's base stands at the top level or inside 'rope_parameters'; of the
        # scaling kinds only the plain one ("default": none) is built
        rope = {}
        for key in ("rope_scaling", "rope_parameters"):
            sub = r.opt_raw(key)
            if sub is None:
                continue
            if not isinstance(sub, dict):
                raise ConfigError(f"config.json: key '{key}' must be an object or null")
            kind = sub.get("rope_type", sub.get("type", "default"))
            if kind != "default":
                raise ConfigError(f"config.json: key '{key}' asks for rope scaling of type "
                                  f"{kind!r}; only 'default' (none) is supported")
            rope.update(sub)
        if "rope_theta" in raw and raw["rope_theta"] is not None:
            theta = r.opt_float("rope_theta", 1e6)
        else:
            theta = KeyReader(rope, "config.json: rope_parameters").opt_float("rope_theta", 1e6)
        if not theta > 0:
            raise ConfigError(f"config.json: key 'rope_theta' must be > 0, got {theta}")
        act = r.opt_str("hidden_act", "silu")
        if act not in ("silu", "gelu_pytorch_tanh"):
            raise ConfigError(f"config.json: key 'hidden_act' must be 'silu' or 'gelu_pytorch_tanh', "
                              f"got {act!r}")
        # no experts (the key absent or 0): every layer has the dense feed-forward; no shared
        # expert (absent or 0): a sparse layer is its routed experts alone
        experts = r.opt_int("num_experts", 0, 0)
        if experts:
            top_k = r.need_int("num_experts_per_tok", 1)
            if top_k > experts:
                raise ConfigError(f"config.json: 'num_experts_per_tok' ({top_k}) exceeds "
                                  f"'num_experts' ({experts})")
            moe_inter = r.need_int("moe_intermediate_size", 1)
        else:
            top_k = r.opt_int("num_experts_per_tok", 0, 0)
            moe_inter = r.opt_int("moe_intermediate_size", 0, 0)
        shared_inter = r.opt_int("shared_expert_intermediate_size", 0, 0)
        sparse_step = r.opt_int("decoder_sparse_step", 1, 1)
        mlp_only = r.opt_int_list("mlp_only_layers", [])
        for l in mlp_only:
            if l >= layers:
                raise ConfigError(f"config.json: 'mlp_only_layers' names layer {l} but the "
                                  f"model has {layers}")
        use_win = r.opt_bool("use_sliding_window", False)
        window = r.opt_int("sliding_window", None, 1)
        max_win_layers = r.opt_int("max_window_layers", 0, 0)
        if use_win and window is None:
            raise ConfigError("config.json: 'use_sliding_window' is true but "
                              "'sliding_window' is missing")
        eos = r.opt_raw("eos_token_id")
        eos = [] if eos is None else eos if isinstance(eos, list) else [eos]
        for e in eos:
            if isinstance(e, bool) or not isinstance(e, int) or e < 0:
                raise ConfigError("config.json: key 'eos_token_id' must be a non-negative "
                                  f"integer or a list of them, got {raw['eos_token_id']!r}")
        return Qwen2MoeConfig(
            vocab_size=vocab, hidden_size=hidden, num_hidden_layers=layers,
            num_attention_heads=heads, num_key_value_heads=kv_heads, head_dim=head_dim,
            intermediate_size=inter, rms_norm_eps=eps, rope_theta=theta,
            tie_word_embeddings=r.opt_bool("tie_word_embeddings", False),
            num_experts=experts, num_experts_per_tok=top_k,
            moe_intermediate_size=moe_inter,
            shared_expert_intermediate_size=shared_inter,
            norm_topk_prob=r.opt_bool("norm_topk_prob", False),
            decoder_sparse_step=sparse_step, mlp_only_layers=mlp_only,
            use_sliding_window=use_win, sliding_window=window,
            max_window_layers=max_win_layers, qkv_bias=r.opt_bool("qkv_bias", True),
            hidden_act=act, eos_token_ids=tuple(eos))
