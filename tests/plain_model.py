"""A plain, slow Qwen2-MoE in 32-bit: whole sequences, no cache, no batching.

Written from the formulas of the reference engine (paths below are relative to
the reference checkout) and, where the reference has no counterpart (q/k/v
bias, sliding window, shared expert, dense layers inside a sparse model,
`norm_topk_prob`), from the architecture's config.json keys. It shares no code
with the engine: it takes the raw config dictionary and a dictionary of
tensors by checkpoint name, and uses only elementary torch operations on CPU.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence, Tuple

import torch

Tensor = torch.Tensor


# --------------------------------------------------------------------------
# parts, one function each
# --------------------------------------------------------------------------
def embedding(tokens: Tensor, table: Tensor) -> Tensor:
    """x[t,:] = table[token[t],:]; no scale, no position term.

    Reference: src/ops/kernels.hip:150-159 (embed_gather_kernel).
    """
    return table[tokens.long()].to(torch.float32)


def rms_norm(x: Tensor, w: Tensor, eps: float) -> Tensor:
    """y = x * rsqrt(mean(x^2) + eps) * w; eps inside the root, gain after.

    Reference: src/ops/kernels.hip:17-41 (sum :23-26, rsqrtf(total/size+eps)
    :34, product :39).
    """
    x = x.to(torch.float32)
    ms = (x * x).sum(dim=-1, keepdim=True) / x.shape[-1]
    return x * torch.rsqrt(ms + eps) * w.to(torch.float32)


def rope_inv_freq(rot_dim: int, theta: float) -> Tensor:
    """f_i = theta^(-2i/D) for i < D/2.

    Reference: src/models/model.hip:635-642. Evaluated in double and rounded
    once to 32-bit.
    """
    vals = [math.pow(float(theta), -(2.0 * i) / rot_dim) for i in range(rot_dim // 2)]
    return torch.tensor(vals, dtype=torch.float64).to(torch.float32)


def apply_rope(x: Tensor, positions: Tensor, theta: float) -> Tensor:
    """Half-split rotation of every head: pairs are (i, i + D/2).

    x'_i = x_i cos(phi) - x_{i+D/2} sin(phi); x'_{i+D/2} = x_i sin(phi) +
    x_{i+D/2} cos(phi); phi = pos * f_i in 32-bit.
    Reference: src/ops/kernels.hip:73-94 (:86-91). x: [T, heads, D].
    """
    d = x.shape[-1]
    half = d // 2
    f = rope_inv_freq(d, theta)
    phi = positions.to(torch.float32)[:, None] * f[None, :]  # [T, half]
    c = torch.cos(phi)[:, None, :]
    s = torch.sin(phi)[:, None, :]
    x1 = x[..., :half]
    x2 = x[..., half:]
    return torch.cat([x1 * c - x2 * s, x1 * s + x2 * c], dim=-1)


def visibility(q_pos: Tensor, k_pos: Tensor, window: Optional[int]) -> Tensor:
    """Key j is visible to query i iff j <= i (causal on absolute positions,
    reference src/ops/attention.hip:216) and, on windowed layers, i - j <
    window."""
    qi = q_pos[:, None]
    kj = k_pos[None, :]
    vis = kj <= qi
    if window is not None:
        vis = vis & ((qi - kj) < window)
    return vis


def attention_core(q: Tensor, k: Tensor, v: Tensor, q_pos: Tensor, k_pos: Tensor,
                   window: Optional[int], slopes: Optional[Sequence[float]] = None) -> Tensor:
    """softmax(q k^T / sqrt(D) + mask) v with grouped heads.

    Query head h reads kv head h // (Hq/Hkv) (consecutive query heads share a
    kv head): reference src/ops/attention.hip:27-28; scale 1/sqrt(D):
    src/models/model.hip:285. q: [Tq,Hq,D]; k, v: [Tk,Hkv,D] -> [Tq,Hq,D].
    `slopes` [Hq] (no counterpart in the reference, whose models rotate): a distance-based
    position bias, slopes[h] * (key position - query position) added to head h's scaled scores.
    """
    tq, hq, d = q.shape
    hkv = k.shape[1]
    group = hq // hkv
    scale = 1.0 / math.sqrt(d)
    vis = visibility(q_pos, k_pos, window)
    out = torch.empty_like(q)
    for h in range(hq):
        g = h // group
        s = (q[:, h, :] @ k[:, g, :].T) * scale
        if slopes is not None:
            s = s + float(slopes[h]) * (k_pos[None, :] - q_pos[:, None]).to(s.dtype)
        s = s.masked_fill(~vis, float("-inf"))
        m = s.max(dim=-1, keepdim=True).values
        p = torch.exp(s - m)
        p = p / p.sum(dim=-1, keepdim=True)
        out[:, h, :] = p @ v[:, g, :]
    return out


def attention_qkv(x: Tensor, w: Dict[str, Tensor], prefix: str, n_heads: int, n_kv: int,
                  head_dim: int, theta: float, positions: Tensor
                  ) -> Tuple[Tensor, Tensor, Tensor]:
    """q, k, v = x W^T + b, split into heads, q and k rotated.

    Weights: reference src/models/model.hip:530-532; the biases are this
    architecture's (the reference loads none) and are added where the weights
    hold them (a model with `qkv_bias` false has none).
    """
    t = x.shape[0]

    def project(name: str) -> Tensor:
        y = x @ w[prefix + name + ".weight"].float().T
        b = w.get(prefix + name + ".bias")
        return y if b is None else y + b.float()

    q, k, v = project("q_proj"), project("k_proj"), project("v_proj")
    q = apply_rope(q.view(t, n_heads, head_dim), positions, theta)
    k = apply_rope(k.view(t, n_kv, head_dim), positions, theta)
    return q, k, v.view(t, n_kv, head_dim)


def gate_activation(g: Tensor, act: str) -> Tensor:
    """silu(z) = z / (1 + exp(-z)) (reference src/ops/kernels.hip:131-140, its only
    activation), or for `hidden_act` = 'gelu_pytorch_tanh' the tanh form of GELU,
    0.5 z (1 + tanh(sqrt(2 / pi) (z + 0.044715 z^3))) (no counterpart in the reference:
    pinned by the library's gelu in tests/test_plain_model.py)."""
    if act == "silu":
        return g / (1.0 + torch.exp(-g))
    if act == "gelu_pytorch_tanh":
        return 0.5 * g * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (g + 0.044715 * g * g * g)))
    raise ValueError(f"hidden_act {act!r}")


def swiglu_mlp(x: Tensor, wg: Tensor, wu: Tensor, wd: Tensor, act: str = "silu",
               biases: Optional[Tuple[Tensor, Tensor, Tensor]] = None) -> Tensor:
    """(act(x Wg^T) * (x Wu^T)) Wd^T; with `biases` (the gate's, the other half's, the down
    product's; the reference has none) each product gets its own added.

    Reference: src/ops/kernels.hip:131-140, src/models/model.hip:313-337.
    """
    g = x @ wg.float().T
    u = x @ wu.float().T
    if biases is not None:
        g, u = g + biases[0].float(), u + biases[1].float()
    y = (gate_activation(g, act) * u) @ wd.float().T
    return y if biases is None else y + biases[2].float()


def router(x: Tensor, wr: Tensor, top_k: int, renorm: bool) -> Tuple[Tensor, Tensor]:
    """softmax over all experts, then the k largest (ties: lower index).

    Reference: src/ops/moe.hip:65-82 (it always renormalises; here only when
    `norm_topk_prob`). Returns ids [T,k] (descending probability) and weights.
    """
    logits = x @ wr.float().T
    m = logits.max(dim=-1, keepdim=True).values
    p = torch.exp(logits - m)
    p = p / p.sum(dim=-1, keepdim=True)
    t, e = p.shape
    ids = torch.empty(t, top_k, dtype=torch.long)
    wts = torch.empty(t, top_k, dtype=torch.float32)
    rows = torch.arange(t)
    work = p.clone()
    for j in range(top_k):
        # a linear scan for the maximum, all rows at once; strictly greater replaces, so among
        # equal probabilities the lowest index stays
        best = torch.zeros(t, dtype=torch.long)
        for c in range(1, e):
            better = work[:, c] > work[rows, best]
            best = torch.where(better, torch.full_like(best, c), best)
        ids[:, j] = best
        wts[:, j] = work[rows, best]
        work[rows, best] = -1.0
    if renorm:
        wts = wts / wts.sum(dim=-1, keepdim=True)
    return ids, wts


def routed_experts(x: Tensor, ids: Tensor, wts: Tensor, w: Dict[str, Tensor],
                   prefix: str, act: str = "silu") -> Tensor:
    """y[t] = sum over selected experts of weight * expert(x[t]).

    Reference: src/models/model.hip:352-433 (gather, per-expert MLP, scale,
    scatter-add); summed here in 32-bit in the order of `ids`.
    """
    t, k = ids.shape
    per = torch.zeros(t, k, x.shape[1], dtype=x.dtype)      # expert output for choice j of row t
    for e in torch.unique(ids).tolist():
        rows, choice = torch.nonzero(ids == e, as_tuple=True)
        p = f"{prefix}experts.{e}."
        per[rows, choice] = swiglu_mlp(x[rows], w[p + "gate_proj.weight"], w[p + "up_proj.weight"],
                                       w[p + "down_proj.weight"], act)
    y = torch.zeros_like(x)
    for j in range(k):                                      # summed in the order of `ids`
        y += wts[:, j:j + 1] * per[:, j]
    return y


def shared_expert(x: Tensor, w: Dict[str, Tensor], prefix: str, act: str = "silu") -> Tensor:
    """sigmoid(x w_gate^T) * mlp_shared(x); one gate scalar per token."""
    s = swiglu_mlp(x, w[prefix + "shared_expert.gate_proj.weight"],
                   w[prefix + "shared_expert.up_proj.weight"],
                   w[prefix + "shared_expert.down_proj.weight"], act)
    gate = x @ w[prefix + "shared_expert_gate.weight"].float().T  # [T,1]
    return s / (1.0 + torch.exp(-gate))


def layer_is_sparse(cfg: dict, layer: int) -> bool:
    """A layer has experts iff it is not in `mlp_only_layers`, the model has
    experts and (layer + 1) is a multiple of `decoder_sparse_step`."""
    if layer in cfg.get("mlp_only_layers", []):
        return False
    step = cfg.get("decoder_sparse_step", 1)
    return cfg.get("num_experts", 0) > 0 and (layer + 1) % step == 0


def layer_window(cfg: dict, layer: int) -> Optional[int]:
    """The window applies to layers with index >= max_window_layers when
    `use_sliding_window` is set."""
    if cfg.get("use_sliding_window", False) and layer >= cfg.get("max_window_layers", 0):
        return int(cfg["sliding_window"])
    return None


def feed_forward(x: Tensor, w: Dict[str, Tensor], cfg: dict, layer: int,
                 probe: Optional[dict] = None) -> Tensor:
    p = f"model.layers.{layer}.mlp."
    act = cfg.get("hidden_act", "silu")
    if not layer_is_sparse(cfg, layer):
        return swiglu_mlp(x, w[p + "gate_proj.weight"], w[p + "up_proj.weight"],
                          w[p + "down_proj.weight"], act)
    if probe is not None:
        probe.setdefault("router_logits", {})[layer] = x @ w[p + "gate.weight"].float().T
    ids, wts = router(x, w[p + "gate.weight"], cfg["num_experts_per_tok"],
                      cfg.get("norm_topk_prob", False))
    y = routed_experts(x, ids, wts, w, p, act)
    if cfg.get("shared_expert_intermediate_size", 0) > 0:
        y = y + shared_expert(x, w, p, act)
    return y


# --------------------------------------------------------------------------
# the whole model
# --------------------------------------------------------------------------
def forward(w: Dict[str, Tensor], cfg: dict, tokens: Sequence[int],
            plan: Optional[List[Tuple[int, Optional[int]]]] = None,
            first_position: int = 0, probe: Optional[dict] = None) -> Tensor:
    """Logits [T, V] of one whole sequence.

    Layer order (pre-norm residual decoder): reference src/models/model.hip:
    1021-1025 and :206-444; final norm and head: :727-755.
    `plan` lists the layers to run as (layer, source): source None means the
    call computes its own keys and values; an integer names an earlier entry of
    the plan whose keys and values it reads instead. Default: each layer once.
    `first_position` shifts all positions (only distances may matter).
    `probe`, if given, receives the router logits of every sparse layer.
    """
    tok = torch.tensor(list(tokens), dtype=torch.long)
    t = tok.shape[0]
    pos = torch.arange(t, dtype=torch.long) + first_position
    hq = cfg["num_attention_heads"]
    hkv = cfg.get("num_key_value_heads", hq)
    d = cfg.get("head_dim", cfg["hidden_size"] // hq)
    theta = cfg.get("rope_theta", 1e6)
    eps = cfg["rms_norm_eps"]
    if plan is None:
        plan = [(i, None) for i in range(cfg["num_hidden_layers"])]
    x = embedding(tok, w["model.embed_tokens.weight"])
    kv_of_call: List[Tuple[Tensor, Tensor]] = []
    for layer, source in plan:
        lp = f"model.layers.{layer}."
        a = rms_norm(x, w[lp + "input_layernorm.weight"], eps)
        q, k, v = attention_qkv(a, w, lp + "self_attn.", hq, hkv, d, theta, pos)
        if source is not None:
            k, v = kv_of_call[source]
        kv_of_call.append((k, v))
        o = attention_core(q, k, v, pos, pos, layer_window(cfg, layer))
        x = x + o.reshape(t, hq * d) @ w[lp + "self_attn.o_proj.weight"].float().T
        m = rms_norm(x, w[lp + "post_attention_layernorm.weight"], eps)
        x = x + feed_forward(m, w, cfg, layer, probe)
    n = rms_norm(x, w["model.norm.weight"], eps)
    head = w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings", False) \
        else w["lm_head.weight"]
    return n @ head.float().T


def greedy_generate(w: Dict[str, Tensor], cfg: dict, prompt: Sequence[int],
                    new_tokens: int) -> List[int]:
    """Greedy continuation, recomputing the whole sequence each time
    (argmax, ties to the lowest id: reference src/runtime/engine.cpp:31-34)."""
    ids = list(prompt)
    out: List[int] = []
    for _ in range(new_tokens):
        logits = forward(w, cfg, ids)
        nxt = int(torch.argmax(logits[-1]))
        out.append(nxt)
        ids.append(nxt)
    return out


# --------------------------------------------------------------------------
# sampling, as the reference's CPU sampler defines it
# --------------------------------------------------------------------------
def sample_distribution(logits: Tensor, temperature: float, top_k: int, top_p: float,
                        repetition_penalty: float, recent: Sequence[int]) -> Tensor:
    """The probability vector the reference's sampler draws from.

    Order: repetition penalty -> /temperature -> top-k -> softmax -> top-p ->
    renormalise (reference src/runtime/engine.cpp:18-72). top_k <= 0 keeps all.
    temperature <= 0 gives a one-hot at the argmax (:31-34).
    """
    l = logits.to(torch.float32).clone()
    v = l.shape[0]
    if repetition_penalty != 1.0:
        for i in recent:  # duplicates are penalised again, as in the reference
            if 0 <= i < v:
                l[i] = l[i] / repetition_penalty if l[i] > 0 else l[i] * repetition_penalty
    if temperature <= 0:
        p = torch.zeros(v)
        p[int(torch.argmax(l))] = 1.0
        return p
    l = l / temperature
    k = v if top_k <= 0 else min(top_k, v)
    order = sorted(range(v), key=lambda i: (-float(l[i]), i))[:k]
    kept = l[order]
    pr = torch.exp(kept - kept[0])
    pr = pr / pr.sum()
    if top_p < 1.0:
        cum = 0.0
        keep = k
        for i in range(k):
            cum += float(pr[i])
            if cum >= top_p:
                keep = i + 1
                break
        order = order[:keep]
        pr = pr[:keep] / pr[:keep].sum()
    p = torch.zeros(v)
    p[order] = pr
    return p
