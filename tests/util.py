"""Helpers shared by the tests: reading a model folder for the plain
implementation, seeded token ids, and the replay schedules (whole, tail,
portions, mixed) expressed as steps of (request, tokens, wanted rows)."""
from __future__ import annotations

import json
import os
import random
from typing import Dict, List, Sequence, Tuple

import torch


def read_folder(model_dir: str) -> Tuple[dict, Dict[str, torch.Tensor]]:
    """config dictionary and name -> 32-bit tensor, read with the safetensors
    package (independent of the engine's own reader)."""
    from safetensors import safe_open
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    tensors = {}
    with safe_open(os.path.join(model_dir, "model.safetensors"), framework="pt") as f:
        for k in f.keys():
            tensors[k] = f.get_tensor(k).to(torch.float32)
    return cfg, tensors


def random_tokens(n: int, vocab: int, seed: int) -> List[int]:
    rng = random.Random(seed)
    return [rng.randrange(vocab) for _ in range(n)]


def routing_margins(w, cfg, tokens) -> torch.Tensor:
    """Per row, the smallest gap between the k-th and (k+1)-th router logit over
    the sparse layers, relative to the largest |logit| of that row and layer."""
    import plain_model
    probe: dict = {}
    plain_model.forward(w, cfg, tokens, probe=probe)
    k = cfg.get("num_experts_per_tok", 0)   # (a model without experts has no routing to tie)
    worst = torch.full((len(tokens),), float("inf"))
    for logits in probe.get("router_logits", {}).values():
        if logits.shape[1] <= k:
            continue
        top = torch.sort(logits, dim=-1, descending=True).values
        gap = (top[:, k - 1] - top[:, k]) / logits.abs().max(dim=-1).values
        worst = torch.minimum(worst, gap)
    return worst


def safe_prompt(w, cfg, n: int, seed: int, rel_margin: float = 0.06,
                max_forwards: int = 0) -> List[int]:
    """Seeded random token ids, redrawn where the plain model's routing would
    be nearly tied: top-k routing is discontinuous, so a row whose k-th and
    (k+1)-th experts are within rounding noise of each other may legitimately
    pick either in reduced precision, and no bound on logits could hold there.
    A row's routing depends only on its prefix, so the prompt grows token by
    token, each drawn again until its own row routes clearly. With
    `max_forwards` the search stops after that many runs of the plain model and
    the prompt found so far (at least two tokens) is returned: with dozens of
    experts in several layers most rows are nearly tied somewhere."""
    rng = random.Random(seed)
    toks: List[int] = []
    forwards = 0
    while len(toks) < n:
        cand = rng.randrange(cfg["vocab_size"])
        forwards += 1
        if float(routing_margins(w, cfg, toks + [cand])[-1]) >= rel_margin:
            toks.append(cand)
        elif max_forwards and forwards >= max_forwards and len(toks) >= 2:
            break
        elif forwards > 60 * n + 200:
            raise RuntimeError("no prompt with clear routing found")
    return toks


# A schedule is a list of steps; a step is (entries, end) with entries
# [(request id, tokens, want rows)] and end = ids finished after the step.
Step = Tuple[List[Tuple[str, List[int], List[int]]], List[str]]


def schedule_whole(rid: str, tokens: Sequence[int]) -> List[Step]:
    return [([(rid, list(tokens), list(range(len(tokens))))], [rid])]


def schedule_tail(rid: str, tokens: Sequence[int], tail: int = 32) -> List[Step]:
    """All but the last min(tail, n-1) tokens in one step, then one by one."""
    n = len(tokens)
    tail = min(tail, n - 1)
    head = n - tail
    steps: List[Step] = [([(rid, list(tokens[:head]), list(range(head)))], [])]
    for i in range(head, n):
        steps.append(([(rid, [tokens[i]], [0])], [rid] if i == n - 1 else []))
    return steps


def schedule_portions(rid: str, tokens: Sequence[int], seed: int = 0) -> List[Step]:
    """Portions of changing size, down to two tokens."""
    sizes = [7, 2, 5, 3, 2, 11, 4, 2, 9]
    rng = random.Random(seed)
    rng.shuffle(sizes)
    steps: List[Step] = []
    i, j, n = 0, 0, len(tokens)
    while i < n:
        m = min(sizes[j % len(sizes)], n - i)
        if n - i - m == 1:   # never leave a single token for the last portion
            m += 1
        j += 1
        steps.append(([(rid, list(tokens[i:i + m]), list(range(m)))], [rid] if i + m == n else []))
        i += m
    return steps


def schedule_mixed(requests: Dict[str, Sequence[int]], seed: int = 0, max_live: int = 4,
                   decode_tail: int = 6) -> List[Step]:
    """Up to `max_live` live requests with staggered starts: prompt portions of
    some beside single tokens of others in the same step. Each request is fed
    in portions (>= 2 tokens) until `decode_tail` tokens remain, which then
    come one per step. Requests start two steps apart; when one ends the next
    waiting one starts, so pages given back are used again."""
    rng = random.Random(seed)
    waiting = list(requests)
    live: Dict[str, int] = {}
    steps: List[Step] = []
    step_no = 0
    while waiting or live:
        if waiting and len(live) < max_live and step_no % 2 == 0:
            live[waiting.pop(0)] = 0
        entries, end = [], []
        for rid in list(live):
            toks = requests[rid]
            done = live[rid]
            left = len(toks) - done
            if left > decode_tail + 1:
                m = min(rng.choice([2, 3, 5, 8, 13]), left - decode_tail)
                if m < 2:
                    m = left - decode_tail
            else:
                m = 1
            if rng.random() < 0.15 and len(live) > 1:
                continue  # a request may be left out of a step and go on later
            entries.append((rid, list(toks[done:done + m]), list(range(m))))
            live[rid] = done + m
            if live[rid] == len(toks):
                end.append(rid)
                del live[rid]
        if entries:
            steps.append((entries, end))
        step_no += 1
    return steps


def schedule_random(requests: Dict[str, Sequence[int]], seed: int, max_live: int = 4) -> List[Step]:
    """A schedule drawn at random: requests start in any order, up to `max_live` live; a live
    request brings 1 to 64 tokens to a step or is left out of it; the entries of a step come
    in any order; logits are wanted at a random subset of the rows."""
    rng = random.Random(seed)
    waiting = list(requests)
    rng.shuffle(waiting)
    live: Dict[str, int] = {}
    steps: List[Step] = []
    while waiting or live:
        while waiting and len(live) < max_live and rng.random() < 0.6:
            live[waiting.pop()] = 0
        entries, end = [], []
        for rid in list(live):
            if rng.random() < 0.2 and len(live) > 1:
                continue
            toks, done = requests[rid], live[rid]
            m = min(len(toks) - done, rng.choice([1, 1, 1, 2, 3, 4, 7, 16, 17, 33, 64]))
            want = sorted(rng.sample(range(m), rng.randint(0, m)))
            entries.append((rid, list(toks[done:done + m]), want))
            live[rid] = done + m
            if live[rid] == len(toks):
                end.append(rid)
                del live[rid]
        if entries:
            rng.shuffle(entries)
            steps.append((entries, end))
    return steps


def run_schedule(runner, steps: List[Step]) -> Dict[str, torch.Tensor]:
    """Feed a schedule through a ModelRunner; returns id -> logits [n, vocab]
    (rows in position order) on the CPU."""
    from ninfer_amd.engine import Chunk
    slots: Dict[str, int] = {}
    rows: Dict[str, List[torch.Tensor]] = {}
    for entries, end in steps:
        chunks = []
        for rid, toks, want in entries:
            if rid not in slots:
                slots[rid] = runner.open()
                rows[rid] = []
            chunks.append(Chunk(slots[rid], toks, want))
        logits = runner.step(chunks)
        o = 0
        for rid, toks, want in entries:
            if want:
                rows[rid].append(logits[o:o + len(want)].float().cpu())
                o += len(want)
        for rid in end:
            runner.close(slots.pop(rid))
    return {rid: torch.cat(v) for rid, v in rows.items()}


class DictSource:
    """A weight source over a dictionary of tensors (for parts built alone)."""

    def __init__(self, tensors: Dict[str, torch.Tensor]):
        self.tensors = tensors

    def shapes(self):
        return {k: tuple(v.shape) for k, v in self.tensors.items()}

    def read(self, name: str) -> torch.Tensor:
        return self.tensors[name]

    def close(self) -> None:
        pass


def random_part_weights(part, seed: int, std: float = 0.2) -> Dict[str, torch.Tensor]:
    """Random 32-bit tensors for everything a part (and its children) expects."""
    from ninfer_amd.weights import RandomSource
    src = RandomSource(part.all_tensor_specs(), seed, torch.float32, std=std)
    return {n: src.read(n) for n in src.specs}


def make_context(ops, act_dtype, seqs, device="cuda"):
    """A StepContext for requests given as (first position, rows)."""
    from ninfer_amd.parts import StepContext
    positions, row_seq, row_start = [], [], []
    for i, (p, q) in enumerate(seqs):
        row_start.append(len(positions))
        positions += list(range(p, p + q))
        row_seq += [i] * q
    row_start.append(len(positions))
    dev = lambda x: torch.tensor(x, dtype=torch.int32, device=device)
    return StepContext(
        ops=ops, act_dtype=act_dtype, device=torch.device(device), T=len(positions), S=len(seqs),
        tokens=dev([0] * len(positions)), positions=dev(positions), row_seq=dev(row_seq),
        seq_slots=dev(list(range(len(seqs)))), seq_row_start=dev(row_start),
        seq_qlen=dev([q for _, q in seqs]), seq_pos0=dev([p for p, _ in seqs]),
        max_qlen=max(q for _, q in seqs), max_kv_len=max(p + q for p, q in seqs),
        all_decode=all(q == 1 for _, q in seqs))


def write_trace(steps: List[Step]) -> str:
    """A schedule as the JSON lines bin/trace_run reads."""
    lines = []
    for i, (entries, end) in enumerate(steps):
        lines.append(json.dumps({"step": i, "entries": [{"id": r, "tokens": t, "want": w}
                                                        for r, t, w in entries], "end": end}))
    return "\n".join(lines) + "\n"


def read_trace_output(out_dir: str, steps: List[Step], vocab: int) -> Dict[str, torch.Tensor]:
    """Logits per request (rows in position order) from the <step>.f32 files."""
    import numpy as np
    rows: Dict[str, List[torch.Tensor]] = {}
    for i, (entries, _) in enumerate(steps):
        wanted = sum(len(w) for _, _, w in entries)
        if not wanted:
            continue
        arr = np.fromfile(os.path.join(out_dir, f"{i}.f32"), dtype="<f4").reshape(wanted, vocab)
        o = 0
        for r, _, w in entries:
            if w:
                rows.setdefault(r, []).append(torch.from_numpy(arr[o:o + len(w)].copy()))
                o += len(w)
    return {k: torch.cat(v) for k, v in rows.items()}


def random_config(seed: int) -> dict:
    """A seeded random configuration of the architecture: head sizes in steps of 16, head
    counts and groups of every kind, widths and vocabularies that are no power of two,
    one expert or many, with and without windows."""
    rng = random.Random(seed)
    nkv = rng.choice([1, 2, 3, 5])
    group = rng.choice([1, 1, 2, 3, 4, 7])
    experts = rng.choice([1, 2, 3, 5, 8, 17, 60, 70])
    window = rng.choice([None, None, 8, 24, 40, 70])
    layers = rng.randint(1, 3)
    cfg = {
        "architectures": ["Qwen2MoeForCausalLM"], "model_type": "qwen2_moe",
        "num_hidden_layers": layers, "hidden_size": rng.choice([48, 64, 72, 96, 100, 128, 136, 160, 200]),
        "num_attention_heads": nkv * group, "num_key_value_heads": nkv,
        "head_dim": rng.choice([16, 32, 48, 64, 80, 96, 112, 128]),
        "intermediate_size": rng.choice([40, 64, 100, 192]),
        "moe_intermediate_size": rng.choice([16, 24, 32, 40, 64, 100]),
        "shared_expert_intermediate_size": rng.choice([16, 48, 64, 96, 130]),
        "num_experts": experts, "num_experts_per_tok": rng.randint(1, min(experts, 6)),
        "norm_topk_prob": rng.random() < 0.5, "decoder_sparse_step": rng.choice([1, 1, 2]),
        "mlp_only_layers": rng.choice([[], [0]]), "vocab_size": rng.choice([97, 256, 333, 1001]),
        "rope_theta": rng.choice([10000.0, 1000000.0]), "use_sliding_window": window is not None,
        "sliding_window": window or 4096, "max_window_layers": rng.randint(0, layers),
        "rms_norm_eps": rng.choice([1e-6, 1e-5]), "tie_word_embeddings": rng.random() < 0.5,
        "hidden_act": "silu", "qkv_bias": rng.random() < 0.75,
    }
    # (drawn last, so that the configurations of earlier seeds stay what they were)
    lacks = rng.random()
    if rng.random() < 0.35:
        cfg["hidden_act"] = "gelu_pytorch_tanh"
    if lacks < 0.15:     # a sparse layer without a shared expert
        del cfg["shared_expert_intermediate_size"]
    elif lacks < 0.22:   # no experts at all: every layer dense
        for key in ("num_experts", "num_experts_per_tok", "moe_intermediate_size",
                    "shared_expert_intermediate_size"):
            del cfg[key]
    return cfg
