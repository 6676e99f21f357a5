"""Toy architectures defined in the tests, to show that parts of other kinds
can be registered, built, loaded and stepped without a change to the
framework's files: a mixer with state of its own; a feed-forward with routing
of its own; another position encoding. They are no models of anyone's.

The mixer keeps one vector of `hidden` numbers per request (fixed size, in the
request's state slot): s <- decay * s + (1 - decay) * x_t for every token in
order, and gives y_t = W s. It keeps nothing in pages.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List

import torch

from ninfer_amd.models.spec import ModelSpec
from ninfer_amd.parts import (Attention, CacheNeed, FeedForward, LMHead, Mixer, NoPosition,
                              PendingRows, PoolSpec, PositionEncoding, PreNormBlock, RMSNorm,
                              RoutedExperts, SwiGLU, TokenEmbedding)
from ninfer_amd.parts.moe import Routing
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
    mlp_bias: bool = False   # the feed-forward's three products each add a bias of the checkpoint
    hidden_act: str = "silu"

    @staticmethod
    def from_dict(raw: dict) -> "ToyConfig":
        return ToyConfig(raw["vocab_size"], raw["hidden_size"], raw["num_hidden_layers"],
                         raw["intermediate_size"], raw["decay"], raw["rms_norm_eps"],
                         raw.get("mlp_bias", False), raw.get("hidden_act", "silu"))


def build_toy(cfg: ToyConfig) -> ModelSpec:
    h = cfg.hidden_size
    emb = TokenEmbedding("embed.", cfg.vocab_size, h)
    blocks = []
    for l in range(cfg.num_hidden_layers):
        p = f"layers.{l}."
        blocks.append(PreNormBlock(RMSNorm(p + "norm1.", h, cfg.rms_norm_eps),
                                   RunningMeanMixer(p, h, cfg.decay),
                                   RMSNorm(p + "norm2.", h, cfg.rms_norm_eps),
                                   SwiGLU(p + "mlp.", h, cfg.intermediate_size, act=cfg.hidden_act,
                                          bias=cfg.mlp_bias)))
    return ModelSpec(emb, blocks, RMSNorm("norm.", h, cfg.rms_norm_eps),
                     LMHead("head.", cfg.vocab_size, h))


def register() -> None:
    register_part("mixer", "running_mean", RunningMeanMixer)
    register_architecture("ToyStateForCausalLM", ToyConfig.from_dict, build_toy)


TOY_CONFIG = {"architectures": ["ToyStateForCausalLM"], "vocab_size": 97, "hidden_size": 40,
              "num_hidden_layers": 2, "intermediate_size": 56, "decay": 0.8, "rms_norm_eps": 1e-5}
# the same with a feed-forward of another kind: the tanh form of GELU as the gate's activation and
# a bias on each of its three products (parameters of the framework's dense feed-forward)
TOY_BIASED_MLP_CONFIG = dict(TOY_CONFIG, mlp_bias=True, hidden_act="gelu_pytorch_tanh")


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
        biases = None
        if cfg.get("mlp_bias"):
            biases = (w[p + "mlp.gate_proj.bias"], w[p + "mlp.up_proj.bias"], w[p + "mlp.down_proj.bias"])
        x = x + pm.swiglu_mlp(m, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"],
                              w[p + "mlp.down_proj.weight"], cfg.get("hidden_act", "silu"), biases)
    return pm.rms_norm(x, w["norm.weight"], cfg["rms_norm_eps"]) @ w["head.weight"].float().T


# ---- a second toy: a feed-forward with routing of its own, another position encoding ----

class HarmonicPosition(PositionEncoding):
    """Rotation by the angles pos * slope / (1 + i), i < rot_dim / 2: no geometric
    series, and only the first rot_dim dims of a head turn; pair i is dims
    (i, i + rot_dim / 2) or, with pairing "interleaved", (2i, 2i + 1)."""

    def __init__(self, rot_dim: int, slope: float, pairing: str = "half"):
        self.rot_dim, self.slope, self.pairing = rot_dim, slope, pairing
        self._table = None

    def inv_freq(self) -> torch.Tensor:
        return torch.tensor([self.slope / (1 + i) for i in range(self.rot_dim // 2)],
                            dtype=torch.float64).to(torch.float32)

    def bind(self, w) -> None:
        self._table = self.inv_freq().to(w.device)

    def table(self):
        return self._table


class BiasedSwitch(FeedForward):
    """Every token goes to the one expert with the largest (logit + bias), where the bias
    is a tensor of the checkpoint; the expert's output is scaled by the softmax weight
    of the biased logits. No shared expert."""

    def __init__(self, prefix: str, hidden: int, inner: int, experts: int):
        self.prefix, self.hidden, self.n = prefix, hidden, experts
        self.experts = RoutedExperts(prefix + "experts.", hidden, inner, experts)
        self.w_router = self.bias = None

    def children(self):
        return [self.experts]

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {self.prefix + "router.weight": TensorSpec((self.n, self.hidden)),
                self.prefix + "router.bias": TensorSpec((self.n,), role="bias")}

    def bind(self, w) -> None:
        self.w_router = w.matrix(self.prefix + "router.weight")
        self.bias = w.float32(self.prefix + "router.bias")

    def forward(self, ctx, x, residual):
        t, e = x.shape[0], self.n
        logits = ctx.empty((t, e), torch.float32)
        ctx.ops.linear(x, self.w_router, logits, bias=self.bias)
        i32 = lambda *shape: ctx.empty(shape, torch.int32)
        r = Routing(i32(t, 1), ctx.empty((t, 1), torch.float32), i32(e + 1), i32(t),
                    i32(min(t, t // 16 + e), 4), i32(t // 256 + e, 4), i32(2))
        ctx.ops.moe_route(logits, e, 1, False, r)
        return PendingRows(self.experts.run(ctx, x, r), r.weights)


class ScoredExperts(FeedForward):
    """Routed experts whose router is not this architecture's: sigmoid scores, a per-expert
    bias of the checkpoint that decides the choice only, a choice limited to the groups of
    experts with the best scores, the chosen weights renormalised and scaled. All of it is
    parameters of the framework's router part and routing kernels; the routing goes with the
    router's product in one together()."""

    def __init__(self, prefix: str, hidden: int, inner: int, experts: int, top_k: int,
                 scale: float, n_group: int = 0, topk_group: int = 0):
        from ninfer_amd.parts.moe import TopKRouter
        self.prefix = prefix
        self.router = TopKRouter(prefix + "router.", hidden, experts, top_k, renorm=True,
                                 score="sigmoid", scale=scale, choice_bias=True,
                                 n_group=n_group, topk_group=topk_group)
        self.experts = RoutedExperts(prefix + "experts.", hidden, inner, experts)

    def children(self):
        return [self.router, self.experts]

    def forward(self, ctx, x, residual):
        with ctx.ops.together():
            routing = self.router.route(ctx, self.router.logits(ctx, x))
        return PendingRows(self.experts.run(ctx, x, routing), routing.weights)


@dataclass
class ToyRoutedConfig:
    raw: dict

    @staticmethod
    def from_dict(raw: dict) -> "ToyRoutedConfig":
        return ToyRoutedConfig(dict(raw))


def build_toy_routed(cfg: ToyRoutedConfig) -> ModelSpec:
    c = cfg.raw
    h = c["hidden_size"]
    blocks = []
    for l in range(c["num_hidden_layers"]):
        p = f"layers.{l}."
        if c.get("positions") == "learned+bias":
            # no rotation: learned absolute positions in the embedding and a distance-based
            # bias on the scores (head i: slope 2^-(i+1)), both parameters of the framework
            attn = Attention(p + "attn.", h, c["heads"], c["kv_heads"], c["head_dim"], NoPosition(),
                             qkv_bias=False, window=c["window"],
                             score_slopes=[2.0 ** -(i + 1) for i in range(c["heads"])],
                             page_size=c.get("page_sizes", [None] * 99)[l])
        else:
            attn = Attention(p + "attn.", h, c["heads"], c["kv_heads"], c["head_dim"],
                             HarmonicPosition(c["rot_dim"], c["slope"], c.get("pairing", "half")),
                             qkv_bias=False,
                             window=c["window"], qk_norm_eps=c.get("qk_norm_eps"))
        if c.get("router") == "scored":
            ff = ScoredExperts(p + "ff.", h, c["inner"], c["experts"], c["top_k"], c["route_scale"],
                               c.get("n_group", 0), c.get("topk_group", 0))
        else:
            ff = BiasedSwitch(p + "ff.", h, c["inner"], c["experts"])
        blocks.append(PreNormBlock(RMSNorm(p + "norm1.", h, c["rms_norm_eps"]), attn,
                                   RMSNorm(p + "norm2.", h, c["rms_norm_eps"]), ff))
    if c.get("positions") == "learned+bias":
        embedding = TokenEmbedding("embed.", c["vocab_size"], h, positions=c["max_positions"],
                                   position_prefix="embed_positions.")
    else:
        embedding = TokenEmbedding("embed.", c["vocab_size"], h)
    return ModelSpec(embedding, blocks,
                     RMSNorm("norm.", h, c["rms_norm_eps"]), LMHead("head.", c["vocab_size"], h))


def register_routed() -> None:
    register_part("position", "harmonic", HarmonicPosition)
    register_part("feed_forward", "biased_switch", BiasedSwitch)
    register_architecture("ToyRoutedForCausalLM", ToyRoutedConfig.from_dict, build_toy_routed)


TOY_ROUTED_CONFIG = {"architectures": ["ToyRoutedForCausalLM"], "vocab_size": 83, "hidden_size": 48,
                     "num_hidden_layers": 2, "heads": 3, "kv_heads": 1, "head_dim": 16, "rot_dim": 8,
                     "slope": 0.7, "window": 11, "inner": 24, "experts": 5, "rms_norm_eps": 1e-5}


TOY_SCORED_CONFIG = dict(TOY_ROUTED_CONFIG, router="scored", top_k=2, route_scale=1.75, experts=6,
                         n_group=3, topk_group=1)

# every query and key head normed over its dims before the rotation
TOY_QK_NORM_CONFIG = dict(TOY_ROUTED_CONFIG, qk_norm_eps=1e-5)

# learned absolute positions (a second gather in the embedding) and a distance-based bias on the
# attention scores instead of a rotation; heads of 64, so that bf16 steps reach the matrix-core
# attention kernels with the bias
TOY_BIASED_CONFIG = dict(TOY_ROUTED_CONFIG, positions="learned+bias", max_positions=160, heads=4,
                         kv_heads=2, head_dim=64, hidden_size=64, window=None)


# the same with pages of another size on each layer (the engine's on the last)
TOY_PAGES_CONFIG = dict(TOY_BIASED_CONFIG, num_hidden_layers=3, page_sizes=[8, 32, None])


def plain_forward_routed(w: Dict[str, torch.Tensor], c: dict, tokens: List[int]) -> torch.Tensor:
    """Whole-sequence reference of the second toy (32-bit, no cache)."""
    import plain_model as pm
    t = len(tokens)
    pos = torch.arange(t)
    hq, hkv, d, rot = c["heads"], c["kv_heads"], c["head_dim"], c["rot_dim"]
    f = torch.tensor([c["slope"] / (1 + i) for i in range(rot // 2)], dtype=torch.float64).float()
    phi = pos.float()[:, None] * f[None, :]
    cos, sin = torch.cos(phi)[:, None, :], torch.sin(phi)[:, None, :]

    def turn(v):   # [T, heads, D]: the first rot dims in pairs, the rest as they are
        if c.get("pairing", "half") == "interleaved":   # pair i = dims (2i, 2i + 1)
            out = v.clone()
            a, b = v[..., 0:rot:2], v[..., 1:rot:2]
            out[..., 0:rot:2] = a * cos - b * sin
            out[..., 1:rot:2] = a * sin + b * cos
            return out
        a, b, rest = v[..., :rot // 2], v[..., rot // 2:rot], v[..., rot:]
        return torch.cat([a * cos - b * sin, a * sin + b * cos, rest], dim=-1)

    x = w["embed.weight"][torch.tensor(tokens)].float()
    slopes = None
    if c.get("positions") == "learned+bias":
        x = x + w["embed_positions.weight"][pos].float()
        slopes = [2.0 ** -(i + 1) for i in range(hq)]
        turn = lambda v: v   # noqa: E731  (no rotation)
    for l in range(c["num_hidden_layers"]):
        p = f"layers.{l}."
        a = pm.rms_norm(x, w[p + "norm1.weight"], c["rms_norm_eps"])
        q = (a @ w[p + "attn.q_proj.weight"].float().T).view(t, hq, d)
        k = (a @ w[p + "attn.k_proj.weight"].float().T).view(t, hkv, d)
        if c.get("qk_norm_eps") is not None:   # every head normed over its dims before it turns
            q = pm.rms_norm(q, w[p + "attn.q_norm.weight"], c["qk_norm_eps"])
            k = pm.rms_norm(k, w[p + "attn.k_norm.weight"], c["qk_norm_eps"])
        q, k = turn(q), turn(k)
        v = (a @ w[p + "attn.v_proj.weight"].float().T).view(t, hkv, d)
        o = pm.attention_core(q, k, v, pos, pos, c["window"], slopes).reshape(t, hq * d)
        x = x + o @ w[p + "attn.o_proj.weight"].float().T
        m = pm.rms_norm(x, w[p + "norm2.weight"], c["rms_norm_eps"])
        y = torch.zeros_like(m)
        if c.get("router") == "scored":
            score = torch.sigmoid(m @ w[p + "ff.router.weight"].float().T)
            biased = score + w[p + "ff.router.choice_bias"].float()
            if c.get("n_group", 0) > 1:
                # only the experts of the topk_group groups with the best biased score are candidates
                per = c["experts"] // c["n_group"]
                best_of = biased.view(t, c["n_group"], per).max(-1).values
                keep = torch.sort(best_of, dim=-1, descending=True, stable=True).indices[:, :c["topk_group"]]
                is_open = torch.zeros_like(best_of, dtype=torch.bool).scatter_(1, keep, True)
                biased = biased.masked_fill(~is_open.repeat_interleave(per, dim=1), float("-inf"))
            for r in range(t):
                # the k largest biased scores (a stable sort: ties to the lower index) choose;
                # the weights are the plain scores of the chosen, renormalised and scaled
                chosen = torch.sort(biased[r], descending=True, stable=True).indices[:c["top_k"]]
                wt = score[r, chosen] / score[r, chosen].sum() * c["route_scale"]
                for e, we in zip(chosen.tolist(), wt.tolist()):
                    pe = f"{p}ff.experts.{e}."
                    y[r] += we * pm.swiglu_mlp(m[r:r + 1], w[pe + "gate_proj.weight"],
                                               w[pe + "up_proj.weight"], w[pe + "down_proj.weight"])[0]
            x = x + y
            continue
        logits = m @ w[p + "ff.router.weight"].float().T + w[p + "ff.router.bias"].float()
        prob = torch.softmax(logits, dim=-1)
        for r in range(t):
            e = int(torch.argmax(prob[r]))        # the first maximum: ties to the lower index
            pe = f"{p}ff.experts.{e}."
            y[r] = prob[r, e] * pm.swiglu_mlp(m[r:r + 1], w[pe + "gate_proj.weight"],
                                              w[pe + "up_proj.weight"], w[pe + "down_proj.weight"])[0]
        x = x + y
    return pm.rms_norm(x, w["norm.weight"], c["rms_norm_eps"]) @ w["head.weight"].float().T


# ---- a third toy: a mixer whose paged cache is not "keys and values of one shape" ----

class LatentMixer(Mixer):
    """Keeps two pools per token that differ in width and in dtype: a latent vector c_t =
    x_t Wc^T of `latent` numbers, always 32-bit, which serves as key and as value, and a short
    position key r_t = x_t Wr^T of `pos_dim` numbers in the activation dtype, turned by the
    angle t * slope in neighbouring pairs. Row t scores key j <= t (within the window) by
    (x_t Wq^T . c_j + turn(x_t Wp^T) . r_j) / sqrt(latent + pos_dim) and returns
    (sum_j p_j c_j) Wo^T. Written with torch operations on the engine's pools and block
    table: what it shows is that the cache manager hands any named pools to a mixer."""

    def __init__(self, prefix: str, hidden: int, latent: int, pos_dim: int, slope: float,
                 window=None, page_size=None):
        self.prefix, self.hidden, self.latent, self.pos_dim = prefix, hidden, latent, pos_dim
        self.slope, self.window, self.page_size = slope, window, page_size
        self.w = {}

    def cache_need(self):
        # (a page size of its own, where the configuration names one: None is the engine's)
        return CacheNeed((PoolSpec("latent", (), (self.latent,), "float32"),
                          PoolSpec("pos_key", (), (self.pos_dim,))), self.window, self.page_size)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        p, h = self.prefix, self.hidden
        return {p + "c.weight": TensorSpec((self.latent, h)), p + "r.weight": TensorSpec((self.pos_dim, h)),
                p + "q.weight": TensorSpec((self.latent, h)), p + "p.weight": TensorSpec((self.pos_dim, h)),
                p + "o.weight": TensorSpec((h, self.latent))}

    def bind(self, w) -> None:
        self.w = {n: w.matrix(self.prefix + n + ".weight").float() for n in "crqpo"}

    def turn(self, v: torch.Tensor, pos: torch.Tensor) -> torch.Tensor:
        phi = pos.float()[:, None] * self.slope
        out = v.clone()
        a, b = v[:, 0::2], v[:, 1::2]
        out[:, 0::2] = a * torch.cos(phi) - b * torch.sin(phi)
        out[:, 1::2] = a * torch.sin(phi) + b * torch.cos(phi)
        return out

    def forward(self, ctx, x, residual, call):
        cache, ps = call.cache, call.cache.page_size
        latent, pos_key = cache["latent"], cache["pos_key"]
        assert latent.dtype == torch.float32 and pos_key.dtype == x.dtype
        assert latent.shape[1:] == (ps, self.latent) and pos_key.shape[1:] == (ps, self.pos_dim)
        xf, pos = x.float(), ctx.positions.long()
        table = cache.block_table.long()[ctx.row_seq.long()]          # [T, pages]
        page = table.gather(1, (pos // ps)[:, None])[:, 0]
        assert (page >= 0).all()
        c = xf @ self.w["c"].T
        latent[page, pos % ps] = c
        pos_key[page, pos % ps] = self.turn(xf @ self.w["r"].T, pos).to(pos_key.dtype)
        q, qp = xf @ self.w["q"].T, self.turn(xf @ self.w["p"].T, pos)
        out = torch.empty_like(c)
        for t in range(x.shape[0]):
            lo = max(0, int(pos[t]) - self.window + 1) if self.window else 0
            js = torch.arange(lo, int(pos[t]) + 1, device=x.device)
            pages = table[t, js // ps]
            assert (pages >= 0).all(), "read of a page that is not held"
            cj, rj = latent[pages, js % ps], pos_key[pages, js % ps].float()
            s = (cj @ q[t] + rj @ qp[t]) / (self.latent + self.pos_dim) ** 0.5
            out[t] = torch.softmax(s, 0) @ cj
        return (out @ self.w["o"].T).to(x.dtype)


def build_toy_latent(cfg: ToyRoutedConfig) -> ModelSpec:
    c = cfg.raw
    h = c["hidden_size"]
    blocks = []
    for l in range(c["num_hidden_layers"]):
        p = f"layers.{l}."
        blocks.append(PreNormBlock(RMSNorm(p + "norm1.", h, c["rms_norm_eps"]),
                                   LatentMixer(p + "mix.", h, c["latent"], c["pos_dim"], c["slope"],
                                               c["windows"][l], c.get("page_sizes", [None] * 99)[l]),
                                   RMSNorm(p + "norm2.", h, c["rms_norm_eps"]),
                                   SwiGLU(p + "mlp.", h, c["inner"])))
    return ModelSpec(TokenEmbedding("embed.", c["vocab_size"], h), blocks,
                     RMSNorm("norm.", h, c["rms_norm_eps"]), LMHead("head.", c["vocab_size"], h))


def register_latent() -> None:
    register_part("mixer", "latent", LatentMixer)
    register_architecture("ToyLatentForCausalLM", ToyRoutedConfig.from_dict, build_toy_latent)


TOY_LATENT_CONFIG = {"architectures": ["ToyLatentForCausalLM"], "vocab_size": 61, "hidden_size": 40,
                     "num_hidden_layers": 2, "latent": 12, "pos_dim": 6, "slope": 0.4,
                     "windows": [None, 9], "inner": 48, "rms_norm_eps": 1e-5}


def plain_forward_latent(w: Dict[str, torch.Tensor], c: dict, tokens: List[int]) -> torch.Tensor:
    """Whole-sequence reference of the third toy (32-bit, no cache)."""
    import plain_model as pm
    t = len(tokens)
    pos = torch.arange(t)
    phi = pos.float()[:, None] * c["slope"]

    def turn(v):
        out = v.clone()
        a, b = v[:, 0::2], v[:, 1::2]
        out[:, 0::2] = a * torch.cos(phi) - b * torch.sin(phi)
        out[:, 1::2] = a * torch.sin(phi) + b * torch.cos(phi)
        return out

    x = w["embed.weight"][torch.tensor(tokens)].float()
    for l in range(c["num_hidden_layers"]):
        p = f"layers.{l}."
        a = pm.rms_norm(x, w[p + "norm1.weight"], c["rms_norm_eps"])
        lat, key = a @ w[p + "mix.c.weight"].T, turn(a @ w[p + "mix.r.weight"].T)
        q, qp = a @ w[p + "mix.q.weight"].T, turn(a @ w[p + "mix.p.weight"].T)
        s = (q @ lat.T + qp @ key.T) / (c["latent"] + c["pos_dim"]) ** 0.5
        dist = pos[:, None] - pos[None, :]
        seen = dist >= 0
        if c["windows"][l]:
            seen &= dist < c["windows"][l]
        s = s.masked_fill(~seen, float("-inf"))
        x = x + (torch.softmax(s, -1) @ lat) @ w[p + "mix.o.weight"].T
        m = pm.rms_norm(x, w[p + "norm2.weight"], c["rms_norm_eps"])
        x = x + pm.swiglu_mlp(m, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"],
                              w[p + "mlp.down_proj.weight"])
    return pm.rms_norm(x, w["norm.weight"], c["rms_norm_eps"]) @ w["head.weight"].float().T
