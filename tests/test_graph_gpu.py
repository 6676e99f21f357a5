"""Decode steps replayed from captured HIP graphs: across the context bounds that key the
graphs (a request grows from one bound into the next while it decodes), and under a cap on
the number of graphs kept. Reference: its single captured decode graph,
src/models/model.hip:786-830, src/runtime/engine.cpp:151-154,186-192."""
import pytest
import torch

import plain_model
import util
from conftest import TINY

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_graph_steps_across_a_context_bound(model_dirs, dtype):
    """Two requests decode from graphs while their contexts pass a bound of the graphs' keys:
    one alone from 1,000 to 1,030 cached tokens (past 1,024), then both, from 1,030 and 2,030
    to 1,070 and 2,070 (past 2,048). One layer sees all keys, the other a window of 40 far
    behind which most of the context lies. Every step equals the same step run eagerly to the
    last bit; in 32-bit the logits are the plain model's."""
    from ninfer_amd import Chunk, EngineOptions, load_model
    d = model_dirs["C"][dtype]
    cfg, w = util.read_folder(d)
    vocab = cfg["vocab_size"]
    # seeds whose routing is clear of 32-bit rounding in every row (margins above 1.5e-4)
    r0, r1 = util.random_tokens(1070, vocab, 15), util.random_tokens(2070, vocab, 8)
    for toks in (r0, r1):
        assert float(util.routing_margins(w, cfg, toks).min()) > 1e-4
    ref0, ref1 = plain_model.forward(w, cfg, r0), plain_model.forward(w, cfg, r1)

    def run(use_graph):
        runner = load_model(d, EngineOptions(dtype=dtype, max_context=2304, prefill_chunk=1024,
                                             num_sequences=2, page_size=16, use_graph=use_graph,
                                             check_pages=True))
        a = runner.open()
        runner.step([Chunk(a, r0[:1000], [])])
        out0, out1 = [], []
        for i in range(1000, 1030):
            out0.append(runner.step([Chunk(a, [r0[i]], [0])])[0].float().cpu())
        b = runner.open()
        runner.step([Chunk(b, r1[:1024], [])])
        runner.step([Chunk(b, r1[1024:2030], [])])
        for i in range(40):
            logits = runner.step([Chunk(b, [r1[2030 + i]], [0]), Chunk(a, [r0[1030 + i]], [0])])
            out1.append(logits[0].float().cpu())
            out0.append(logits[1].float().cpu())
        return runner, torch.stack(out0), torch.stack(out1)

    eager, e0, e1 = run(False)
    graphs, g0, g1 = run(True)
    assert not eager._graphs
    assert set(graphs._graphs) == {(1, 1024), (1, 2048), (2, 2048), (2, 2304)}
    assert all(e["graph"] is not None for e in graphs._graphs.values())
    assert torch.equal(g0, e0) and torch.equal(g1, e1)
    assert any(g.window_freed > 100 for g in graphs.cache.groups)
    if dtype == "float32":
        torch.testing.assert_close(g0, ref0[1000:1070], atol=2e-5, rtol=1e-4)
        torch.testing.assert_close(g1, ref1[2030:2070], atol=2e-5, rtol=1e-4)
    else:
        # Random tokens: in bfloat16 some row's routing is nearly tied and may go either
        # way, which no bound on single logits survives. The typical row is near the plain
        # model's, and far nearer than to the logits of the position before.
        for got, ref, first in ((g0, ref0, 1000), (g1, ref1, 2030)):
            err = (got - ref[first:first + len(got)]).abs().max(-1).values
            off = (got - ref[first - 1:first - 1 + len(got)]).abs().max(-1).values
            assert float(err.median()) < 0.06 and float(err.median()) < float(off.median()) / 5


@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("C", "bfloat16")])
def test_the_graph_cache_is_capped(model_dirs, name, dtype):
    """Under the scheduler the number of requests in a decode step walks up and down (1 ... 8
    ... 1 here), each count a graph of its own. With a cap of three the least recently
    replayed graphs go, never more than three are kept, dropped shapes are captured again
    when they come back, and the tokens are those of the run without graphs."""
    from ninfer_amd import EngineOptions, Request, SamplingParams, Scheduler, load_model
    from ninfer_amd.sampling import Sampler
    d = model_dirs[name][dtype]
    vocab = TINY[name][0]["vocab_size"]
    prompts = [util.random_tokens(3 + 2 * i, vocab, 300 + i) for i in range(8)]
    news = [40, 6, 34, 10, 28, 14, 22, 18]

    def run(use_graph, max_graphs):
        runner = load_model(d, EngineOptions(dtype=dtype, max_context=96, num_sequences=8,
                                             page_size=8, prefill_chunk=8, use_graph=use_graph,
                                             max_graphs=max_graphs))
        sched = Scheduler(runner, Sampler(runner.ops, runner.device))
        reqs = [Request(f"q{i}", list(p), SamplingParams.greedy(m), [])
                for i, (p, m) in enumerate(zip(prompts, news))]
        seen = 0
        for r in reqs:
            sched.add(r)
        while sched.has_work():
            sched.step()
            seen = max(seen, len(runner._graphs))
        assert all(r.status == "finished" for r in reqs)
        return runner, [r.output for r in reqs], seen

    _, want, _ = run(False, 3)
    free, got_all, shapes = run(True, 32)
    assert got_all == want and free.graphs_dropped == 0
    assert shapes >= 6, "the count of requests in a decode step took many values"
    capped, got, seen = run(True, 3)
    assert got == want
    assert seen <= 3 and len(capped._graphs) <= 3
    assert capped.graphs_dropped >= shapes - 3, "every shape went through the three places"


def test_close_gives_the_device_memory_back():
    """An engine at the benchmark's layer sizes (two layers) that has decoded from captured
    graphs: after close() its weights, cache, graphs' pools and the kernels' workspaces are
    back with the device, so that another engine can take its place (the command line's
    --verify builds the 32-bit engine after closing the first)."""
    import gc
    import ninfer_amd
    from bench import MODELS
    raw = dict(MODELS["a2.7b"][1], num_hidden_layers=2)
    gc.collect()
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    before = torch.cuda.memory_allocated()
    eng = ninfer_amd.Ninfer(random_config=raw, random_seed=3, max_context=256, prefill_chunk=128,
                            num_sequences=4, use_graph=True)
    held = torch.cuda.memory_allocated() - before
    assert held > 3e9, "two layers, the embedding and the head are several GB"
    prompts = [util.random_tokens(n, raw["vocab_size"], n) for n in (40, 9, 130)]
    outs = eng.generate(prompts, ninfer_amd.SamplingParams.greedy(12), stop_ids=[])
    assert all(len(o) == 12 for o in outs)
    assert any(e["graph"] is not None for e in eng.runner._graphs.values())
    eng.close()
    after = torch.cuda.memory_allocated()
    assert after - before < 8 << 20, f"{(after - before) >> 20} MiB still held after close()"
    assert torch.cuda.memory_reserved() - after < 64 << 20, "the allocator's cache was emptied"


def test_verify_at_benchmark_layer_sizes(tmp_path):
    """The command line's --verify with two layers at the benchmark's layer sizes and decode
    steps from graphs: the bfloat16 engine is closed and its memory is back before the 32-bit
    engine with the same (bf16-rounded) weights is built, and the report is made."""
    import json
    import os
    import re
    import subprocess
    import sys
    from bench import MODELS
    from conftest import ROOT
    raw = dict(MODELS["a2.7b"][1], num_hidden_layers=2)
    with open(tmp_path / "config.json", "w") as f:
        json.dump(raw, f)
    proc = subprocess.run(
        [sys.executable, os.path.join(ROOT, "bin", "ninfer"), str(tmp_path), "--random-weights", "5",
         "--random-prompts", "20,33", "--max-new", "8", "--temperature", "0", "--repeat-penalty",
         "1", "--max-context", "256", "--max-seqs", "2", "--graph", "--verify"],
        capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    held = re.search(r"first engine is closed, (\d+) MiB", proc.stderr)
    # (what stays is torch's workspace for the vendor library's products, 76 MiB, which the
    # process keeps; the engine itself held several GB)
    assert held and int(held.group(1)) < 100, proc.stderr[-1000:]
    report = [l for l in proc.stderr.splitlines() if "verify:" in l and "closed" not in l]
    assert len(report) >= 1 and ("PASS" in report[-1] or "parts from the 32-bit output" in report[-1])
    assert len(proc.stdout.strip().splitlines()) == 2
