"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

The default run has the layer sizes of Qwen1.5-MoE-A2.7B (24 layers, hidden
2048, 16 heads of 128, 60 experts top-4 of 1408, shared expert 5632, vocabulary
151936) with random bf16 weights generated on the device, a batch of 8
requests and a context of 8192 tokens each (the cache is filled with random
keys and values; token ids are seeded random). A step is one decode step: one
new token for every request of the batch through the engine's step function
(replayed from a captured HIP graph unless --no-graph) and its device sampler. One JSON line is printed: decoded tokens a second as
`value`; the 2,048-token prefill under "prefill"; the decode step's memory
roofline under "roofline" (with the rate of a plain read of HBM measured beside it, and the
step's fraction of that); decode at batch 1 and 64 under "points"; and under
"graph_check" the largest difference between replayed and eager decode steps at
those batches (untimed; 0.0 when the replays are exact).
Peaks: HBM 8 TB/s; dense bf16 MFMA 2.5 PFLOP/s (fp32 157.3 TFLOP/s).

    python bench.py --scenario long [--model 57b-a14b] [--requests 8] [--prompt 32768] [--new 256]

is another measurement with a JSON line of its own: the scheduler serves
`--requests` concurrent requests with random prompts of `--prompt` tokens,
prefilled in portions of 2,048 tokens interleaved with the decoding of the
others, `--new` tokens each, sampled at temperature 0.7 from fixed seeds.
"""
import argparse
import json
import sys
import time

HBM_PEAK = 8.0e12
FLOP_PEAK = {"bfloat16": 2.5e15, "float32": 157.3e12}

CONFIG_C = {
    "architectures": ["Qwen2MoeForCausalLM"], "model_type": "qwen2_moe",
    "num_hidden_layers": 24, "hidden_size": 2048, "num_attention_heads": 16,
    "num_key_value_heads": 16, "head_dim": 128, "intermediate_size": 5632,
    "moe_intermediate_size": 1408, "shared_expert_intermediate_size": 5632,
    "num_experts": 60, "num_experts_per_tok": 4, "norm_topk_prob": False,
    "decoder_sparse_step": 1, "mlp_only_layers": [], "vocab_size": 151936,
    "rope_theta": 1000000.0, "use_sliding_window": False, "rms_norm_eps": 1e-6,
    "tie_word_embeddings": False, "hidden_act": "silu",
}


CONFIG_D = dict(CONFIG_C, num_hidden_layers=28, hidden_size=3584, num_attention_heads=28,
                num_key_value_heads=4, intermediate_size=18944, moe_intermediate_size=2560,
                shared_expert_intermediate_size=20480, num_experts=64, num_experts_per_tok=8)
MODELS = {"a2.7b": ("Qwen1.5-MoE-A2.7B", CONFIG_C), "57b-a14b": ("Qwen2-57B-A14B", CONFIG_D)}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=8192)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the model has")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--no-points", action="store_true", help="skip batch 1 and 64")
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--no-check", action="store_true",
                    help="skip the comparison of replayed with eager decode steps (untimed)")
    ap.add_argument("--prefill-tokens", type=int, default=2048,
                    help="length of the timed prefill (the contract's figure is at 2,048)")
    ap.add_argument("--graph", dest="graph", action="store_true", default=True,
                    help="decode steps replayed from a captured HIP graph (the default)")
    ap.add_argument("--no-graph", dest="graph", action="store_false",
                    help="every decode step launched kernel by kernel")
    ap.add_argument("--model", default="a2.7b", choices=sorted(MODELS),
                    help="layer sizes: a2.7b (the default and the headline) or 57b-a14b")
    ap.add_argument("--profile", action="store_true",
                    help="also time every kind of kernel call of one eager decode step and one "
                         "prefill with device events, with the bytes and flops of each kind, its "
                         "floor and the fraction of it reached (untimed runs of their own; the "
                         "table goes to stderr and under \"profile\")")
    ap.add_argument("--scenario", default="decode", choices=["decode", "long"])
    ap.add_argument("--requests", type=int, default=8, help="--scenario long: concurrent requests")
    ap.add_argument("--prompt", type=int, default=32768, help="--scenario long: prompt tokens")
    ap.add_argument("--new", type=int, default=256, help="--scenario long: new tokens a request")
    ap.add_argument("--portion", type=int, default=2048,
                    help="--scenario long: the scheduler's token budget of a step")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2

    import torch
    import ninfer_amd
    from ninfer_amd import Chunk, EngineOptions, random_model
    from ninfer_amd.parts.moe import SparseMoE
    from ninfer_amd.sampling import SampleRow, Sampler, SamplingParams
    from collections import Counter

    model_name, model_cfg = MODELS[args.model]
    raw = dict(model_cfg)
    layers_full = raw["num_hidden_layers"]
    if args.layers:
        raw["num_hidden_layers"] = args.layers
    L = raw["num_hidden_layers"]
    H, Hq, Hkv, D = raw["hidden_size"], raw["num_attention_heads"], raw["num_key_value_heads"], \
        raw["head_dim"]
    Im, Is, E, k, V = raw["moe_intermediate_size"], raw["shared_expert_intermediate_size"], \
        raw["num_experts"], raw["num_experts_per_tok"], raw["vocab_size"]
    esize = 2 if args.dtype == "bfloat16" else 4
    page = 16
    if args.scenario == "long":
        return long_scenario(args, raw, model_name, layers_full)
    max_b = args.batch if args.no_points else max(args.batch, 64)
    ctx = args.context
    opt = EngineOptions(dtype=args.dtype, max_context=ctx, prefill_chunk=max(args.prefill_tokens, max_b),
                        num_sequences=max_b, page_size=page, use_graph=args.graph)
    t0 = time.time()
    runner = random_model(raw, 1234, opt)
    torch.cuda.synchronize()
    print(f"[bench] model ready in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
    for pools in runner.cache.pools.values():   # a cache full of synthetic keys and values
        for pool in pools.values():
            pool.normal_()
    sampler = Sampler(runner.ops, runner.device)
    gen = torch.Generator().manual_seed(7)
    greedy = SamplingParams.greedy()
    moes = [b.feed_forward for b in runner.spec.blocks if isinstance(b.feed_forward, SparseMoE)]

    def decode_run(batch: int, steps: int, warmup: int):
        start = ctx - (steps + warmup) - 1
        slots = [runner.open() for _ in range(batch)]
        for s in slots:                       # positions 0..start-1 count as cached
            runner.cache.reserve(s, start)
            runner.cache.commit(s, start)
        toks = torch.randint(0, V, (batch,), generator=gen).tolist()
        rows = [SampleRow(greedy, Counter(), i, 0, 1) for i in range(batch)]

        def one():
            nonlocal toks
            logits = runner.step([Chunk(s, [t], [0]) for s, t in zip(slots, toks)])
            toks = sampler.sample(logits, rows)

        for _ in range(warmup):
            one()
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(steps):
            one()
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t) / steps
        distinct = [int(torch.unique(m.last_ids).numel()) for m in moes if m.last_ids is not None]
        for s in slots:
            runner.close(s)
        n_exp = sum(distinct) / max(len(distinct), 1)
        per_layer = ((Hq + 2 * Hkv) * D * H + H * Hq * D + E * H + n_exp * 3 * Im * H
                     + 3 * Is * H + H) * esize
        kv = batch * 2 * L * Hkv * D * (ctx - steps / 2) * esize
        nbytes = L * per_layer + V * H * esize + kv
        return dt, nbytes, n_exp

    def prefill_run(T: int, reps: int):
        toks = torch.randint(0, V, (T,), generator=gen).tolist()
        times = []
        for _ in range(reps + 2):
            s = runner.open()
            torch.cuda.synchronize()
            t = time.perf_counter()
            runner.step([Chunk(s, toks, [T - 1])])
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t)
            runner.close(s)
        dt = sorted(times[2:])[len(times[2:]) // 2]
        print(f"[bench] prefill of {T} tokens, ms: " + " ".join(f"{x * 1e3:.2f}" for x in times)
              + " (the first two are warm-up; the median of the rest counts)", file=sys.stderr, flush=True)
        flops = T * 2 * L * ((Hq + 2 * Hkv) * D * H + Hq * D * H + E * H + k * 3 * Im * H
                             + 3 * Is * H + H) + L * 2 * Hq * D * T * T + 2 * V * H
        return dt, flops

    def graph_check(batch: int) -> float:
        """Replayed steps against the same steps launched kernel by kernel, at this batch (so
        with the same library products inside the graph): `batch` requests with a real
        64-token prompt each, then four decode steps of fixed tokens, once with replays and
        once with the graphs forgotten before every step (the first step of a shape runs
        eagerly, under the same context bound as its graph), with an eager step of another
        shape between the replays. Largest difference of any logit (0.0: replays are exact)."""
        prompts = [torch.randint(0, V, (64,), generator=gen).tolist() for _ in range(batch)]
        feed = [torch.randint(0, V, (batch,), generator=gen).tolist() for _ in range(4)]
        outs = []
        for replay in (True, False):
            runner._graphs.clear()
            slots = [runner.open() for _ in range(batch)]
            for i in range(0, batch, 16):
                runner.step([Chunk(s, p, []) for s, p in zip(slots[i:i + 16], prompts[i:i + 16])])
            got = []
            for n, toks in enumerate(feed):
                if not replay:
                    runner._graphs.clear()
                logits = runner.step([Chunk(s, [t], [0]) for s, t in zip(slots, toks)])
                got.append(logits.float().clone())
                if n == 1 and batch < max_b:
                    extra = runner.open()
                    runner.step([Chunk(extra, prompts[0][:9], [8])])
                    runner.close(extra)
            outs.append(got)
            for s in slots:
                runner.close(s)
        runner._graphs.clear()
        return max(float((a - b).abs().max()) for a, b in zip(*outs))

    def call_cost(name, a, kw):
        """What one call of the kernel library has to move and to compute, from its own
        arguments: a function, evaluated after the step (it may read device tensors such as
        the experts' offsets), that returns (bytes, flops). Bytes: every operand read once and
        every result written once (weights of experts that got rows only; the cached keys and
        values a request's rows can see, once per request); flops: two per multiply-add."""
        def nbytes(*ts):
            return sum(t.numel() * t.element_size() for t in ts if t is not None)

        def product(x_rows, x, w_rows, w, out_rows, out_cols, out):
            k_ = x.shape[1]
            return (x_rows * k_ * x.element_size() + w_rows * k_ * w.element_size()
                    + out_rows * out_cols * out.element_size(), 2.0 * x_rows * w_rows * k_)

        def grouped(x, w, offsets, n_rows, out):
            def cost():
                counts = (offsets[1:] - offsets[:-1]).cpu()
                used = int((counts > 0).sum())
                per_expert = w.shape[1] * w.shape[2]
                return (used * per_expert * w.element_size() + n_rows * x.shape[1] * x.element_size()
                        + nbytes(out), 2.0 * n_rows * per_expert)
            return cost

        if name == "linear":
            x, w, out = a[0], a[1], a[2]
            return lambda: product(x.shape[0], x, w.shape[0], w, out.shape[0], out.shape[1], out)
        if name == "swiglu_linear":
            x, w, out = a[0], a[1], a[2]
            return lambda: product(x.shape[0], x, w.shape[0], w, out.shape[0], out.shape[1], out)
        if name == "qkv_rope":
            x, w, qkv = a[0], a[1], a[3]
            return lambda: product(x.shape[0], x, w.shape[0], w, qkv.shape[0], qkv.shape[1], qkv)
        if name == "grouped_swiglu":
            return grouped(a[0], a[1], a[2], a[3].shape[0], a[5])
        if name == "grouped_down":
            return grouped(a[0], a[1], a[2], a[3].shape[0], a[4])
        if name == "paged_attention":
            qkv, k_pool, sctx, n_q, n_kv, d, window = a[0], a[1], a[4], a[5], a[6], a[7], a[9]
            out = kw.get("out", a[11] if len(a) > 11 else None)

            def cost():
                pos = sctx.positions.cpu().tolist()
                seq = sctx.row_seq.cpu().tolist()
                seen = [min(p + 1, window) if window else p + 1 for p in pos]
                keys = {}
                for s_, p, n_ in zip(seq, pos, seen):     # keys a request's rows see, all told
                    lo, hi = keys.get(s_, (p - n_ + 1, p))
                    keys[s_] = (min(lo, p - n_ + 1), max(hi, p))
                kv = sum(hi - lo + 1 for lo, hi in keys.values()) * 2 * n_kv * d * k_pool.element_size()
                return (kv + len(pos) * n_q * d * qkv.element_size() + nbytes(out),
                        4.0 * n_q * d * sum(seen))
            return cost
        if name == "rmsnorm":
            x, out = a[0], a[3]
            rs = kw.get("rows_sum")
            extra = nbytes(kw.get("delta")) + (nbytes(rs.y, rs.shared) if rs is not None else 0)
            touched = out.shape[0] * x.shape[1] * 4
            return lambda: (2 * touched + nbytes(out) + extra, 0.0)   # residual read and written
        if name == "_launch_held":
            def cost():
                total_b = total_f = 0.0
                for g, keep in a[0]:
                    x, w, out, offsets = keep[0], keep[1], keep[2], keep[4]
                    w_rows = g.N * (2 if g.epilogue else 1)
                    if offsets is None:
                        b_, f_ = product(g.M, x, w_rows, w, g.M, g.N, out)
                    else:
                        counts = (offsets[1:] - offsets[:-1]).cpu()
                        used = int((counts > 0).sum())
                        b_ = (used * w_rows * g.K * w.element_size() + g.M * g.K * x.element_size()
                              + g.M * g.N * out.element_size())
                        f_ = 2.0 * g.M * w_rows * g.K
                    total_b += b_
                    total_f += f_
                return total_b, total_f
            return cost
        tensors = [t for t in list(a) + list(kw.values()) if isinstance(t, torch.Tensor)]
        if name in ("embed",):      # a gather: the rows read, not the table
            return lambda: (2 * nbytes(a[2]), 0.0)
        if name in ("rope_kv_write",):   # q and k rotated in place, k and v written to pages
            return lambda: (2 * nbytes(a[0]), 0.0)
        return lambda: (nbytes(*[t for t in tensors if t.numel() < (1 << 28)]), 0.0)

    def profile_calls(label: str, chunks) -> dict:
        """One eager step by kind of kernel call: microseconds (every call of the kernel
        library is bracketed by device events; calls inside `together()` are launched when it
        ends and are timed there, as one kind), the bytes and flops the calls have to move
        and compute (`call_cost`), their floor max(bytes / 8 TB/s, flops / peak) and the
        fraction floor / time; the floors add up to the step's. Everything runs on one stream
        here (a long portion's shared expert otherwise runs beside the routed path, and times
        would overlap). The reference prints its table of times per phase
        (src/models/model.hip:1066-1081)."""
        ops = runner.ops
        spans = []
        one_stream, ops.beside_min_rows = ops.beside_min_rows, 1 << 30

        def kind(name, a):
            if name in ("linear", "swiglu_linear"):
                return f"{name} {a[0].shape[0]}x{a[1].shape[1]}->{a[2].shape[1]}"
            if name in ("grouped_swiglu", "grouped_down"):
                return f"{name} {a[0].shape[0]} rows"
            return name

        names = ["embed", "rmsnorm", "qkv_rope", "rope_kv_write", "paged_attention", "linear",
                 "swiglu_linear", "grouped_swiglu", "grouped_down", "moe_route",
                 "moe_combine", "_launch_held"]
        saved = {n: getattr(ops, n) for n in names}

        depth = [0]

        def wrap(n):
            def call(*a, **kw):
                if depth[0]:
                    return saved[n](*a, **kw)       # part of a call that is timed
                # inside `together()` a call is either held back (it is launched, and timed,
                # when the block ends) or runs at once (the vendor library's products do)
                waiting = (len(ops._held), ops._held_route) if ops._held is not None else None
                s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                cost = call_cost(n, a, kw)
                s.record()
                depth[0] += 1
                try:
                    out = saved[n](*a, **kw)
                finally:
                    depth[0] -= 1
                e.record()
                if waiting is not None and ops._held is not None \
                        and (len(ops._held), ops._held_route) != waiting:
                    return out                      # held back
                spans.append(("products launched together" if n == "_launch_held" else kind(n, a),
                              s, e, cost))
                return out
            return call

        use_graph, runner.options.use_graph = runner.options.use_graph, False
        try:
            for n in names:
                setattr(ops, n, wrap(n))
            runner.step(chunks)
            torch.cuda.synchronize()
        finally:
            for n in names:
                setattr(ops, n, saved[n])
            runner.options.use_graph = use_graph
            ops.beside_min_rows = one_stream
        peak = FLOP_PEAK[args.dtype]
        table = {}
        for k_, s, e, cost in spans:
            b_, f_ = cost()
            row = table.setdefault(k_, [0, 0.0, 0.0, 0.0, 0.0])
            row[0] += 1
            row[1] += s.elapsed_time(e) * 1e3
            row[2] += b_
            row[3] += f_
            row[4] += max(b_ / HBM_PEAK, f_ / peak) * 1e6
        total = sum(r[1] for r in table.values())
        floor = sum(r[4] for r in table.values())
        print(f"[bench] {label}: {total:.0f} us in kernel calls (eager, with event overhead); "
              f"floor {floor:.0f} us = {floor / total:.3f} of it", file=sys.stderr)
        print(f"[bench]   {'us':>9} {'%':>5} {'calls':>5} {'MB':>9} {'GFLOP':>9} {'floor us':>9} "
              f"{'frac':>5}  kind", file=sys.stderr)
        for k_, (calls, us, b_, f_, fl) in sorted(table.items(), key=lambda kv: -kv[1][1]):
            print(f"[bench]   {us:9.1f} {100 * us / total:5.1f} {calls:5d} {b_ / 1e6:9.1f} "
                  f"{f_ / 1e9:9.1f} {fl:9.1f} {fl / us:5.2f}  {k_}", file=sys.stderr)
        out = {k_: {"us": round(us, 1), "mb": round(b_ / 1e6, 1), "gflop": round(f_ / 1e9, 1),
                    "floor_us": round(fl, 1), "frac": round(fl / us, 3)}
               for k_, (_, us, b_, f_, fl) in table.items()}
        out["step"] = {"us": round(total, 1), "floor_us": round(floor, 1),
                       "frac": round(floor / total, 3)}
        return out

    def read_rate() -> float:
        """Bytes a second at which a kernel that only reads streams 4 GiB from HBM (the
        library's read probe: 16-byte non-temporal loads, nothing written): what the memory
        system gives a decode step's weights and cache at best."""
        src = torch.empty(1 << 30, dtype=torch.float32, device=runner.device).normal_()
        for _ in range(2):
            runner.ops.read_probe(src)
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(5):
            runner.ops.read_probe(src)
        torch.cuda.synchronize()
        return 5 * src.numel() * 4 / (time.perf_counter() - t)

    dt, nbytes, n_exp = decode_run(args.batch, args.steps, args.warmup)
    result = {
        "metric": f"decode tok/s at batch {args.batch} ({model_name} shapes, context {ctx})",
        "value": round(args.batch / dt, 2), "unit": "tok/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(dt * 1e3, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic",
        "config": {"model": f"{model_name} shapes, random weights", "global_batch": args.batch,
                   "seq_len": ctx, "parallelism": "single GPU", "layers": L,
                   "layers_full": layers_full, "hidden": H, "heads": Hq, "kv_heads": Hkv,
                   "head_dim": D, "moe_intermediate": Im, "shared_intermediate": Is,
                   "intermediate": raw["intermediate_size"], "experts": E, "top_k": k, "vocab": V,
                   "page_size": page, "graph": bool(args.graph)},
        "roofline": {"bound": "hbm", "achieved": round(nbytes / dt / 1e9, 1),
                     "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": round(nbytes / dt / HBM_PEAK, 4),
                     "distinct_experts_per_layer": round(n_exp, 1)},
    }
    plain_read = read_rate()
    result["roofline"]["measured_read"] = round(plain_read / 1e9, 1)
    result["roofline"]["frac_of_read"] = round(nbytes / dt / plain_read, 4)
    if not args.no_prefill:
        pt = min(args.prefill_tokens, ctx)
        pdt, flops = prefill_run(pt, 5)
        result["prefill"] = {"value": round(pt / pdt, 1), "tokens": pt,
                             "ms": round(pdt * 1e3, 3),
                             "frac": round(flops / pdt / FLOP_PEAK[args.dtype], 4)}
    if not args.no_points:
        points, fracs = {}, {}
        for b in (1, 64):
            steps = max(8, args.steps // (4 if b == 64 else 1))
            d, nb, _ = decode_run(b, steps, max(2, args.warmup // 2))
            points[f"decode_b{b}"] = round(b / d, 2)
            fracs[f"decode_b{b}"] = round(nb / d / HBM_PEAK, 4)
        result["points"] = points
        result["points_hbm_frac"] = fracs   # the same roofline as the default step's, per point
    if args.profile:
        slots = [runner.open() for _ in range(args.batch)]
        for sl in slots:
            runner.cache.reserve(sl, ctx - 2)
            runner.cache.commit(sl, ctx - 2)
        toks = torch.randint(0, V, (args.batch,), generator=gen).tolist()
        step = [Chunk(sl, [t], [0]) for sl, t in zip(slots, toks)]
        profile_calls("warm-up", step)
        result["profile"] = {"decode": profile_calls(f"decode step, batch {args.batch}", step)}
        for sl in slots:
            runner.close(sl)
        pt = min(args.prefill_tokens, ctx)
        ptoks = torch.randint(0, V, (pt,), generator=gen).tolist()
        for label in ("warm-up", f"prefill of {pt} tokens"):
            sl = runner.open()
            table = profile_calls(label, [Chunk(sl, ptoks, [pt - 1])])
            runner.close(sl)
        result["profile"]["prefill"] = table
    if args.graph and not args.no_check:
        batches = [args.batch] if args.no_points else sorted({1, args.batch, 64})
        worst = max(graph_check(b) for b in batches)
        result["graph_check"] = {"batches": batches, "max_abs_diff": worst}
        if worst != 0.0:
            print(f"[bench] WARNING: replayed steps differ from eager steps by {worst}",
                  file=sys.stderr, flush=True)
    print(json.dumps(result), flush=True)
    return 0


def long_scenario(args, raw, model_name, layers_full) -> int:
    """Long prompts through the scheduler: portions of prompts beside decode tokens."""
    import torch
    from ninfer_amd import EngineOptions, Request, Scheduler, random_model
    from ninfer_amd.sampling import Sampler, SamplingParams

    n, plen, new = args.requests, args.prompt, args.new
    page, chunk = 16, args.portion
    ctx = -(-(plen + new) // page) * page
    opt = EngineOptions(dtype=args.dtype, max_context=ctx, prefill_chunk=chunk, num_sequences=n,
                        page_size=page, use_graph=args.graph)
    t0 = time.time()
    runner = random_model(raw, 1234, opt)
    torch.cuda.synchronize()
    print(f"[bench] model ready in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
    sampler = Sampler(runner.ops, runner.device)
    gen = torch.Generator().manual_seed(11)
    V = raw["vocab_size"]

    def serve(n_req, prompt_len, new_tokens):
        sched = Scheduler(runner, sampler, max_batch_tokens=chunk, max_seqs=n_req)
        reqs = [Request(id=f"r{i}", prompt=torch.randint(0, V, (prompt_len,), generator=gen).tolist(),
                        params=SamplingParams(temperature=0.7, seed=100 + i, max_new_tokens=new_tokens))
                for i in range(n_req)]
        for r in reqs:
            sched.add(r)
        torch.cuda.synchronize()
        t = time.perf_counter()
        last = t
        while sched.has_work():
            sched.step()
            if time.perf_counter() - last > 20:
                last = time.perf_counter()
                fed = sum(r.cached for r in reqs if r.status == "running")
                print(f"[bench] step {sched.steps}: {fed} tokens cached by running requests, "
                      f"{len(sched.finished)} finished", file=sys.stderr, flush=True)
        torch.cuda.synchronize()
        return time.perf_counter() - t, sched, reqs

    serve(min(n, 2), 3 * chunk // 2, 4)                     # warm-up: every kind of step once
    dt, sched, reqs = serve(n, plen, new)
    generated = sum(len(r.output) for r in reqs)
    failed = [r.id for r in reqs if r.status != "finished"]
    print(json.dumps({
        "metric": f"long-context serving ({model_name} shapes): {n} x {plen}-token prompts in "
                  f"{chunk}-token portions interleaved with decode, {new} new tokens each",
        "value": round((n * plen + generated) / dt, 1), "unit": "tok/s (prompt + generated)",
        "seconds": round(dt, 3), "steps": sched.steps,
        "prompt_tokens": n * plen, "generated_tokens": generated,
        "preemptions": sum(r.preemptions for r in reqs), "failed": failed,
        "n_gpus": 1, "higher_is_better": True, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic", "config": {"model": f"{model_name} shapes, random weights",
                                        "layers": raw["num_hidden_layers"], "layers_full": layers_full,
                                        "requests": n, "prompt": plen, "new_tokens": new,
                                        "portion": chunk, "page_size": page, "temperature": 0.7,
                                        "graph": bool(args.graph)}}), flush=True)
    return 1 if failed else 0


if __name__ == "__main__":
    sys.exit(main())
