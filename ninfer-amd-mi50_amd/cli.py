"""Command line in the reference's manner: `ninfer <model_dir> [options]`
(src/apps/ninfer.cpp:55-119). Option names and meanings are the reference's
where it has them: --max-context, --prefill-chunk, --max-new, --temperature
(0 = greedy), --top-k, --top-p, --repeat-penalty, --seed,
--graph, --verify (here against the 32-bit path), --log-level. Prompts are token ids (there is no tokenizer here):
--prompt-ids, --prompt-file, --random-prompts. Generated ids go to stdout, one
line per request; diagnostics go to stderr (src/apps/ninfer.cpp:1-2). An
unknown option is an error (:114-116). Without a prompt it is the reference's
interactive loop (:222-233): every line of standard input is a turn of token
ids, the answer is generated from all turns and answers so far, until the
input ends. A one-shot run with --seed 0 samples from the fixed seed 1234, as
the reference's does (:205); the loop draws a seed per turn.
"""
from __future__ import annotations

import argparse
import json
import random
import sys
import time
from typing import List, Optional


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(prog="ninfer", description="generation with a model folder's architecture on one MI355X")
    ap.add_argument("model_dir", help="folder with config.json (and model.safetensors)")
    ap.add_argument("--prompt-ids", action="append", default=[],
                    help="a prompt as comma-separated token ids (may be given several times)")
    ap.add_argument("--prompt-file", help="JSON file: a list of lists of token ids")
    ap.add_argument("--random-prompts", help="comma-separated lengths of seeded random prompts")
    ap.add_argument("--max-context", type=int, default=32768, help="KV capacity in tokens per request")
    ap.add_argument("--prefill-chunk", type=int, default=512, help="token budget of one step")
    ap.add_argument("--max-new", type=int, default=512, help="new tokens per generation")
    ap.add_argument("--temperature", type=float, default=0.7, help="sampling temperature (0 = greedy)")
    ap.add_argument("--top-k", type=int, default=50)
    ap.add_argument("--top-p", type=float, default=0.95)
    ap.add_argument("--repeat-penalty", type=float, default=1.05)
    ap.add_argument("--seed", type=int, default=0, help="sampling seed (0: 1234 for a one-shot run, a fresh one per turn of the loop)")
    ap.add_argument("--graph", action="store_true", help="replay decode steps from a HIP graph")
    ap.add_argument("--verify", action="store_true",
                    help="generate again in the 32-bit path and report where the outputs part")
    ap.add_argument("--log-level", choices=["debug", "info", "warn", "error"], default="info")
    ap.add_argument("--dtype", choices=["bf16", "fp32", "bfloat16", "float32"], default="bf16")
    ap.add_argument("--random-weights", type=int, metavar="SEED",
                    help="fill the model with seeded random weights (needs only config.json)")
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--kv-pages", type=int, help="pages per cache group")
    ap.add_argument("--kv-gib", type=float, help="size of the paged cache over all layers, in GiB "
                    "(instead of --kv-pages; default: room for --max-seqs requests of --max-context)")
    ap.add_argument("--max-seqs", type=int, default=8, help="most live requests")
    ap.add_argument("--eos-id", type=int, help="stop token (default: config.json eos_token_id)")
    return ap


def main(argv: Optional[List[str]] = None) -> int:
    args = build_parser().parse_args(argv)
    quiet = args.log_level in ("warn", "error")

    def log(msg: str) -> None:
        if not quiet:
            print(f"[ninfer] {msg}", file=sys.stderr, flush=True)

    from .api.ninfer import Ninfer
    from .config.base import read_config_json
    from .sampling.params import SamplingParams

    dtype = {"bf16": "bfloat16", "fp32": "float32"}.get(args.dtype, args.dtype)
    raw = read_config_json(args.model_dir)
    prompts: List[List[int]] = [[int(x) for x in p.split(",") if x.strip()]
                                for p in args.prompt_ids]
    if args.prompt_file:
        with open(args.prompt_file) as f:
            prompts += [list(map(int, p)) for p in json.load(f)]
    if args.kv_pages is not None and args.kv_gib is not None:
        print("ninfer: error: give --kv-pages or --kv-gib, not both", file=sys.stderr)
        return 1
    t0 = time.time()
    common = dict(max_context=args.max_context, prefill_chunk=args.prefill_chunk,
                  num_sequences=args.max_seqs, dtype=dtype, page_size=args.page_size,
                  num_pages=args.kv_pages, use_graph=args.graph,
                  kv_bytes=int(args.kv_gib * (1 << 30)) if args.kv_gib is not None else None)
    try:
        if args.random_weights is not None:
            eng = Ninfer(random_config=raw, random_seed=args.random_weights, **common)
        else:
            eng = Ninfer(args.model_dir, **common)
        if args.random_prompts:   # the vocabulary is the bound model's, whatever its config calls it
            rng = random.Random(args.seed or 1234)
            for n in args.random_prompts.split(","):
                prompts.append([rng.randrange(eng.vocab) for _ in range(int(n))])
        log(f"engine ready in {time.time() - t0:.1f} s: vocab={eng.vocab} ctx={args.max_context} "
            f"chunk={args.prefill_chunk} seqs={args.max_seqs} dtype={dtype}")
        stop = [args.eos_id] if args.eos_id is not None else None
        if not prompts:
            return _interactive(eng, args, stop)
        params = SamplingParams(args.temperature, args.top_k, args.top_p, args.repeat_penalty,
                                args.seed or 1234, args.max_new)
        t1 = time.time()
        outs = eng.generate(prompts, params, stop)
        dt = time.time() - t1
        for o in outs:
            print(",".join(map(str, o)))
        n = sum(len(o) for o in outs)
        log(f"{n} tokens in {dt:.2f} s ({n / max(dt, 1e-9):.1f} tok/s)")
        if args.verify:
            eng.close()   # the golden engine takes the first one's place: never both at once
            del eng
            import torch
            log(f"verify: the first engine is closed, {torch.cuda.memory_allocated() >> 20} MiB "
                f"of device memory still held")
            _verify(args, raw, common, prompts, params, stop, outs)
    except Exception as e:  # the reference exits 1 with the message (src/apps/ninfer.cpp:234-237)
        print(f"ninfer: error: {e}", file=sys.stderr)
        return 1
    return 0


def _verify(args, raw, common, prompts, params, stop, outs) -> None:
    """The reference's --verify runs the prompt again on one GPU as the golden output and
    reports where the two-GPU output parts from it (src/apps/ninfer.cpp:137-176). Here the
    golden run is the 32-bit path of the same model, with the same sampling seed."""
    from .api.ninfer import Ninfer
    if common["dtype"] == "float32":
        print("[ninfer] verify: the run was in 32-bit already", file=sys.stderr)
        return
    golden = dict(common, dtype="float32", use_graph=False)
    if golden.get("num_pages") is None and golden.get("kv_bytes") is None:
        # the 32-bit cache takes twice the bytes per token: room for these prompts is enough
        per = max(len(p) for p in prompts) + params.max_new_tokens
        golden["num_pages"] = (-(-per // golden["page_size"]) + 1) * min(len(prompts),
                                                                        golden["num_sequences"])
    if args.random_weights is not None:   # the same values, rounded as the first run's were
        eng = Ninfer(random_config=raw, random_seed=args.random_weights,
                     random_weights_dtype=common["dtype"], **golden)
    else:
        eng = Ninfer(args.model_dir, **golden)
    want = eng.generate(prompts, params, stop)
    same = True
    for r, (a, b) in enumerate(zip(outs, want)):
        if a != b:
            same = False
            i = next((j for j, (x, y) in enumerate(zip(a, b)) if x != y), min(len(a), len(b)))
            print(f"[ninfer] verify: request {r} parts from the 32-bit output at token {i} "
                  f"({len(a)} / {len(b)} tokens); rounding noise of bfloat16 is expected where "
                  f"two tokens are nearly as likely", file=sys.stderr)
    if same:
        print(f"[ninfer] verify: PASS, the outputs equal the 32-bit path's "
              f"({sum(len(o) for o in outs)} tokens)", file=sys.stderr)


def _interactive(eng, args, stop) -> int:
    """Turn after turn from standard input: a line of comma-separated token ids is added to
    what has been said, the answer is generated from all of it and added too."""
    from .sampling.params import SamplingParams
    print("ninfer ready: one line of comma-separated token ids per turn, end of input to exit",
          file=sys.stderr, flush=True)
    said: List[int] = []
    for line in sys.stdin:
        ids = [int(x) for x in line.replace(",", " ").split()]
        if not ids:
            continue
        said += ids
        params = SamplingParams(args.temperature, args.top_k, args.top_p, args.repeat_penalty,
                                args.seed, args.max_new)
        answer = eng.generate([said], params, stop)[0]
        print(",".join(map(str, answer)), flush=True)
        said += answer
    return 0


if __name__ == "__main__":
    sys.exit(main())
