"""A toy architecture defined in the tests, to show that a mixer with state of
its own can be registered, built, loaded and stepped without a change to the
framework's files. It is no model of anyone's.

The mixer keeps one vector of `hidden` numbers per request (fixed size, in the
request's state slot): s <- decay * s + (1 - decay) * x_t for every token in
order, and gives y_t = W s. It keeps nothing in pages.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List

import torch

from ninfer_amd.models.spec import ModelSpec
from ninfer_amd.parts import (LMHead, Mixer, PreNormBlock, RMSNorm, SwiGLU, TokenEmbedding)
from ninfer_amd.registry import register_architecture, register_part
from ninfer_amd.weights import TensorSpec


class RunningMeanMixer(Mixer):
    def __init__(self, prefix: str, hidden: int, decay: float):
        self.prefix, self.hidden, self.decay = prefix, hidden, decay
        self.w = None

    def state_floats(self) -> int:
        return self.hidden

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {self.prefix + "mix.weight": TensorSpec((self.hidden, self.hidden))}

    def bind(self, w) -> None:
        self.w = w.matrix(self.prefix + "mix.weight")

    def forward(self, ctx, x, residual, call):
        out = torch.empty_like(x)
        slots = ctx.seq_slots.tolist()
        starts = ctx.seq_row_start.tolist()
        for i, slot in enumerate(slots):
            s = call.state[slot].clone()
            for r in range(starts[i], starts[i + 1]):
                s = self.decay * s + (1 - self.decay) * x[r].float()
                out[r] = (self.w.float() @ s).to(x.dtype)
            call.state[slot] = s
        return out


@dataclass
class ToyConfig:
    vocab_size: int
    hidden_size: int
    num_hidden_layers: int
    intermediate_size: int
    decay: float
    rms_norm_eps: float

    @staticmethod
    def from_dict(raw: dict) -> "ToyConfig":
        return ToyConfig(raw["vocab_size"], raw["hidden_size"], raw["num_hidden_layers"],
                         raw["intermediate_size"], raw["decay"], raw["rms_norm_eps"])


def build_toy(cfg: ToyConfig) -> ModelSpec:
    h = cfg.hidden_size
    emb = TokenEmbedding("embed.", cfg.vocab_size, h)
    blocks = []
    for l in range(cfg.num_hidden_layers):
        p = f"layers.{l}."
        blocks.append(PreNormBlock(RMSNorm(p + "norm1.", h, cfg.rms_norm_eps),
                                   RunningMeanMixer(p, h, cfg.decay),
                                   RMSNorm(p + "norm2.", h, cfg.rms_norm_eps),
                                   SwiGLU(p + "mlp.", h, cfg.intermediate_size)))
    return ModelSpec(emb, blocks, RMSNorm("norm.", h, cfg.rms_norm_eps),
                     LMHead("head.", cfg.vocab_size, h))


def register() -> None:
    register_part("mixer", "running_mean", RunningMeanMixer)
    register_architecture("ToyStateForCausalLM", ToyConfig.from_dict, build_toy)


TOY_CONFIG = {"architectures": ["ToyStateForCausalLM"], "vocab_size": 97, "hidden_size": 40,
              "num_hidden_layers": 2, "intermediate_size": 56, "decay": 0.8, "rms_norm_eps": 1e-5}


def plain_forward(w: Dict[str, torch.Tensor], cfg: dict, tokens: List[int]) -> torch.Tensor:
    """Whole-sequence reference of the toy model (32-bit, no cache, no state)."""
    import plain_model as pm
    x = w["embed.weight"][torch.tensor(tokens)].float()
    for l in range(cfg["num_hidden_layers"]):
        p = f"layers.{l}."
        a = pm.rms_norm(x, w[p + "norm1.weight"], cfg["rms_norm_eps"])
        s = torch.zeros(cfg["hidden_size"])
        y = torch.empty_like(a)
        for t in range(a.shape[0]):
            s = cfg["decay"] * s + (1 - cfg["decay"]) * a[t]
            y[t] = w[p + "mix.weight"].float() @ s
        x = x + y
        m = pm.rms_norm(x, w[p + "norm2.weight"], cfg["rms_norm_eps"])
        x = x + pm.swiglu_mlp(m, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"],
                              w[p + "mlp.down_proj.weight"])
    return pm.rms_norm(x, w["norm.weight"], cfg["rms_norm_eps"]) @ w["head.weight"].float().T
