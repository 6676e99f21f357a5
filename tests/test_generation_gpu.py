"""Generation through the entry points on the GPU: greedy tokens equal the
plain implementation's; long decoding; the first tokens of a sequence; the
command line; the toy architecture and other layer plans with the real
kernels."""
import os
import subprocess
import sys

import pytest
import torch

import plain_model
import toy
import util
from conftest import ROOT, TINY

pytestmark = pytest.mark.gpu


def test_greedy_generation_through_the_entry_point(model_dirs):
    import ninfer_amd
    for name in ("A", "B"):
        d = model_dirs[name]["float32"]
        cfg, w = util.read_folder(d)
        eng = ninfer_amd.Ninfer(d, max_context=96, prefill_chunk=16, num_sequences=3,
                                dtype="float32", page_size=8)
        prompts = [util.random_tokens(n, cfg["vocab_size"], 40 + n) for n in (5, 11, 17, 30)]
        outs = eng.generate(prompts, ninfer_amd.SamplingParams.greedy(8), stop_ids=[])
        for p, o in zip(prompts, outs):
            assert o == plain_model.greedy_generate(w, cfg, p, 8)
        assert eng.kv_pages()["free"] == eng.kv_pages()["total"]


@pytest.mark.parametrize("seed", range(10))
def test_a_crowd_under_a_tight_pool_generates_what_each_request_does_alone(model_dirs, seed):
    """32-bit, requests drawn at random, greedy or at a temperature: through a scheduler with
    few slots and a pool that just fits the largest request (so requests are preempted and
    recomputed), every request gets the tokens it gets alone. Its random numbers are named by
    its seed and id, not by its place in the queue."""
    import random
    from ninfer_amd import EngineOptions, Request, SamplingParams, Scheduler, load_model
    from ninfer_amd.sampling import Sampler
    rng = random.Random(seed)
    name = "ABC"[seed % 3]
    d = model_dirs[name]["float32"]
    vocab = TINY[name][0]["vocab_size"]
    n = rng.randint(3, 8)
    prompts = [util.random_tokens(rng.randint(1, 60), vocab, seed * 50 + i) for i in range(n)]
    news = [rng.randint(1, 24) for _ in range(n)]
    temp = 0.8 if seed % 2 else 0.0

    def requests():
        return [Request(f"q{i}", list(p), SamplingParams(temperature=temp, top_k=0, top_p=1.0,
                                                         repetition_penalty=1.0, seed=7 + i % 2,
                                                         max_new_tokens=m), [])
                for i, (p, m) in enumerate(zip(prompts, news))]

    alone = load_model(d, EngineOptions(dtype="float32", max_context=96, num_sequences=1,
                                        page_size=16, prefill_chunk=64))
    sampler = Sampler(alone.ops, alone.device)
    want = []
    for r in reversed(requests()):        # one scheduler each, in another order
        s = Scheduler(alone, sampler)
        s.add(r)
        s.run()
        want.insert(0, r.output)
    page = rng.choice([4, 8, 16])
    pages = max(-(-(len(p) + m) // page) for p, m in zip(prompts, news)) + rng.randint(0, 4)
    runner = load_model(d, EngineOptions(dtype="float32", max_context=96, num_sequences=3,
                                         page_size=page, num_pages=pages,
                                         prefill_chunk=rng.choice([8, 16, 64]),
                                         poison_freed_pages=True, check_pages=True, use_graph=seed % 3 == 0))
    sched = Scheduler(runner, Sampler(runner.ops, runner.device))
    crowd = requests()
    for r in crowd:
        sched.add(r)
    sched.run()
    for r, w in zip(crowd, want):
        assert r.status == "finished" and r.output == w, f"{name} seed {seed}: {r.id}"
    if temp > 0:   # requests that share a seed still draw their own numbers
        assert len({tuple(o[:4]) for o in want if len(o) >= 4}) > 1
    runner.cache.check()
    assert all(g.allocator.in_use == 0 for g in runner.cache.groups)


def test_sessions_like_the_reference_binding(model_dirs):
    import ninfer_amd
    d = model_dirs["A"]["float32"]
    cfg, w = util.read_folder(d)
    eng = ninfer_amd.Ninfer(d, max_context=64, prefill_chunk=4, num_sequences=2, dtype="float32")
    toks = util.random_tokens(14, cfg["vocab_size"], 9)
    ref = plain_model.forward(w, cfg, toks)
    with eng.session() as s, eng.session() as t:
        l1 = s.prefill(toks[:9])                       # cut into portions of 4 inside
        assert s.length == 9 and l1.shape == (cfg["vocab_size"],)
        torch.testing.assert_close(torch.from_numpy(l1), ref[8], atol=2e-5, rtol=1e-4)
        t.prefill(toks[:3])
        both = eng.decode_batch([s, t], [toks[9], toks[3]])
        torch.testing.assert_close(torch.from_numpy(both[0]), ref[9], atol=2e-5, rtol=1e-4)
        torch.testing.assert_close(torch.from_numpy(both[1]), ref[3], atol=2e-5, rtol=1e-4)
        assert eng.sample(l1, temperature=0.0) == int(ref[8].argmax())
        drawn = {eng.sample(l1, temperature=1.0, top_k=5, top_p=1.0, seed=sd) for sd in range(1, 40)}
        assert drawn <= set(ref[8].topk(5).indices.tolist()) and len(drawn) > 1
        s.reset()
        assert s.length == 0
    assert eng.vocab == cfg["vocab_size"] and eng.kv_bytes_per_token == 2 * 2 * 2 * 16 * 4


def test_long_decoding_and_first_tokens(model_dirs):
    """300 tokens decoded one by one after a one-token prompt (first tokens of a
    sequence, many page edges, the window passing pages) equal the whole-sequence
    logits of the plain implementation."""
    from ninfer_amd import Chunk, EngineOptions, load_model
    for dtype in ("float32", "bfloat16"):
        d = model_dirs["B"][dtype]
        cfg, w = util.read_folder(d)
        _, w16 = util.read_folder(model_dirs["B"]["bfloat16"])
        toks = util.safe_prompt(w16, cfg, 300, 4242)
        ref = plain_model.forward(w, cfg, toks)
        runner = load_model(d, EngineOptions(dtype=dtype, max_context=320, num_sequences=1,
                                             page_size=16))
        s = runner.open()
        rows = [runner.step([Chunk(s, [t], [0])])[0].float().cpu() for t in toks]
        got = torch.stack(rows)
        bound = dict(atol=3e-5, rtol=1e-4) if dtype == "float32" else dict(atol=6e-2, rtol=5e-2)
        torch.testing.assert_close(got, ref, **bound)
        assert runner.cache.groups[1].window_freed >= (300 - 24) // 16


def test_command_line(model_dirs):
    d = model_dirs["A"]["float32"]
    cfg, w = util.read_folder(d)
    prompt = util.random_tokens(7, cfg["vocab_size"], 3)
    proc = subprocess.run(
        [sys.executable, os.path.join(ROOT, "bin", "ninfer"), d, "--prompt-ids",
         ",".join(map(str, prompt)), "--random-prompts", "5,9", "--max-new", "6", "--temperature",
         "0", "--dtype", "fp32", "--max-context", "64", "--prefill-chunk", "8", "--seed", "3",
         "--repeat-penalty", "1"],
        capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    lines = proc.stdout.strip().splitlines()
    assert len(lines) == 3
    assert [int(x) for x in lines[0].split(",")] == plain_model.greedy_generate(w, cfg, prompt, 6)
    # without a prompt: turns from standard input, each answered from everything said so far
    second = util.random_tokens(4, cfg["vocab_size"], 4)
    turns = ",".join(map(str, prompt)) + "\n\n" + " ".join(map(str, second)) + "\n"
    proc = subprocess.run(
        [sys.executable, os.path.join(ROOT, "bin", "ninfer"), d, "--max-new", "5", "--temperature",
         "0", "--dtype", "fp32", "--max-context", "64", "--eos-id", "-1", "--repeat-penalty", "1"],
        input=turns, capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    answers = [[int(x) for x in l.split(",")] for l in proc.stdout.strip().splitlines()]
    first = plain_model.greedy_generate(w, cfg, prompt, 5)
    assert answers == [first, plain_model.greedy_generate(w, cfg, prompt + first + second, 5)]
    # --verify: the same prompts again in the 32-bit path, and a line that says how they compare
    proc = subprocess.run(
        [sys.executable, os.path.join(ROOT, "bin", "ninfer"), model_dirs["A"]["bfloat16"],
         "--prompt-ids", ",".join(map(str, prompt)), "--max-new", "4", "--temperature", "0",
         "--max-context", "64", "--repeat-penalty", "1", "--kv-gib", "0.001", "--verify"],
        capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    # what --verify has to say follows from the run's own output and the plain model on the
    # same (bfloat16-rounded) weights, which is what the 32-bit path computes
    _, w16 = util.read_folder(model_dirs["A"]["bfloat16"])
    out = [int(x) for x in proc.stdout.strip().splitlines()[0].split(",")]
    want = plain_model.greedy_generate(w16, cfg, prompt, 4)
    report = [l for l in proc.stderr.splitlines() if "verify:" in l and "is closed" not in l]
    assert len(report) == 1
    if out == want:
        assert "PASS" in report[0] and "(4 tokens)" in report[0]
    else:
        first = next(i for i, (a, b) in enumerate(zip(out, want)) if a != b)
        assert f"request 0 parts from the 32-bit output at token {first} " in report[0]
    bad = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "ninfer"), d, "--no-such-flag"],
                         capture_output=True, text=True, timeout=120)
    assert bad.returncode != 0


def test_verify_names_the_first_token_that_differs(model_dirs, capsys):
    """--verify's report on a case with a known answer: outputs that were made to differ from
    the 32-bit path's at chosen places."""
    from ninfer_amd import SamplingParams, cli
    d = model_dirs["A"]["bfloat16"]
    cfg, w16 = util.read_folder(d)
    prompts = [util.random_tokens(n, cfg["vocab_size"], 8 + n) for n in (6, 9, 4)]
    golden = [plain_model.greedy_generate(w16, cfg, p, 5) for p in prompts]
    args = cli.build_parser().parse_args([d])
    common = dict(max_context=64, prefill_chunk=16, num_sequences=4, dtype="bfloat16",
                  page_size=16, num_pages=None, use_graph=False, kv_bytes=None)
    params = SamplingParams.greedy(5)
    cli._verify(args, cfg, common, prompts, params, None, [list(g) for g in golden])
    err = capsys.readouterr().err
    assert "verify: PASS" in err and "(15 tokens)" in err
    outs = [list(g) for g in golden]
    outs[1][3] = (outs[1][3] + 1) % cfg["vocab_size"]
    outs[2] = outs[2][:2]
    cli._verify(args, cfg, common, prompts, params, None, outs)
    err = capsys.readouterr().err
    assert "PASS" not in err
    assert "request 1 parts from the 32-bit output at token 3 (5 / 5 tokens)" in err
    assert "request 2 parts from the 32-bit output at token 2 (2 / 5 tokens)" in err
    assert "request 0" not in err


def test_toy_mixer_on_the_gpu(tmp_path):
    import ninfer_amd
    from ninfer_amd import EngineOptions, load_model
    toy.register()
    d = str(tmp_path / "toy")
    ninfer_amd.write_random_model(d, toy.TOY_CONFIG, 5, std=0.2)
    cfg, w = util.read_folder(d)
    runner = load_model(d, EngineOptions(dtype="float32", max_context=64, num_sequences=3))
    reqs = {f"t{i}": util.random_tokens(n, 97, 60 + i) for i, n in enumerate([9, 21, 14, 30])}
    ref = {k: toy.plain_forward(w, cfg, v) for k, v in reqs.items()}
    got = util.run_schedule(runner, util.schedule_mixed(reqs, seed=3, max_live=3))
    for k in reqs:
        torch.testing.assert_close(got[k], ref[k], atol=2e-5, rtol=1e-4)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_feed_forward_with_biases_and_another_activation_on_the_gpu(tmp_path, dtype):
    """A dense feed-forward with GELU's tanh form as the gate's activation and a bias on each of
    its three products, on the product kernels' epilogues (few rows and portions)."""
    import ninfer_amd
    from ninfer_amd import EngineOptions, load_model
    toy.register()
    cfg = toy.TOY_BIASED_MLP_CONFIG
    d = str(tmp_path / "toy_biased_mlp")
    ninfer_amd.write_random_model(d, cfg, 6, dtype=dtype, std=0.2)
    _, w = util.read_folder(d)
    runner = load_model(d, EngineOptions(dtype=dtype, max_context=64, num_sequences=3))
    reqs = {f"t{i}": util.random_tokens(n, 97, 90 + i) for i, n in enumerate([9, 21, 14, 50])}
    ref = {k: toy.plain_forward(w, cfg, v) for k, v in reqs.items()}
    got = util.run_schedule(runner, util.schedule_mixed(reqs, seed=3, max_live=3))
    whole = util.run_schedule(runner, util.schedule_whole("t3", reqs["t3"]))["t3"]
    for k in reqs:
        if dtype == "float32":
            torch.testing.assert_close(got[k], ref[k], atol=2e-5, rtol=1e-4)
        else:
            assert float((got[k] - ref[k]).abs().max()) < 0.04 * float(ref[k].abs().max())
    if dtype == "float32":
        torch.testing.assert_close(whole, ref["t3"], atol=2e-5, rtol=1e-4)
    else:
        assert float((whole - ref["t3"]).abs().max()) < 0.04 * float(ref["t3"].abs().max())
        no_bias = toy.plain_forward(w, dict(cfg, mlp_bias=False), reqs["t3"])
        assert float((whole - ref["t3"]).abs().max()) < float((whole - no_bias).abs().max()) / 3


def test_toy_routed_feed_forward_and_position_on_the_gpu(tmp_path):
    """The second toy (a routed feed-forward with a router bias, another position
    encoding with a partial rotation, a window) on the kernels, 32-bit."""
    import ninfer_amd
    from ninfer_amd import EngineOptions, load_model
    toy.register_routed()
    d = str(tmp_path / "toy_routed")
    ninfer_amd.write_random_model(d, toy.TOY_ROUTED_CONFIG, 9, std=0.3)
    cfg, w = util.read_folder(d)
    runner = load_model(d, EngineOptions(dtype="float32", max_context=64, num_sequences=3,
                                         page_size=4))
    reqs = {f"r{i}": util.random_tokens(n, 83, 40 + i) for i, n in enumerate([7, 26, 15, 33])}
    ref = {k: toy.plain_forward_routed(w, cfg, v) for k, v in reqs.items()}
    got = util.run_schedule(runner, util.schedule_mixed(reqs, seed=4, max_live=3))
    for k in reqs:
        torch.testing.assert_close(got[k], ref[k], atol=3e-5, rtol=1e-4)
    k0 = "r1"
    torch.testing.assert_close(
        util.run_schedule(runner, util.schedule_tail(k0, reqs[k0], 6))[k0], ref[k0],
        atol=3e-5, rtol=1e-4)


def test_toy_router_with_other_scores_on_the_gpu(tmp_path):
    """The toy whose router has sigmoid scores, a choice bias, renormalised and scaled weights:
    parameters of the routing kernels, also where the block that computes a decode step's
    router logits routes the rows itself. 32-bit against the plain model; bfloat16 (the fused
    launch of few rows) against the 32-bit engine on the same bf16-rounded weights, on rows
    that route alike."""
    import ninfer_amd
    from ninfer_amd import EngineOptions, load_model
    toy.register_routed()
    d = str(tmp_path / "toy_scored")
    ninfer_amd.write_random_model(d, toy.TOY_SCORED_CONFIG, 12, std=0.3)
    cfg, w = util.read_folder(d)
    runner = load_model(d, EngineOptions(dtype="float32", max_context=64, num_sequences=3,
                                         page_size=4, check_pages=True))
    reqs = {f"r{i}": util.random_tokens(n, 83, 60 + i) for i, n in enumerate([7, 26, 15, 33])}
    ref = {k: toy.plain_forward_routed(w, cfg, v) for k, v in reqs.items()}
    got = util.run_schedule(runner, util.schedule_mixed(reqs, seed=4, max_live=3))
    for k in reqs:
        torch.testing.assert_close(got[k], ref[k], atol=3e-5, rtol=1e-4)
    torch.testing.assert_close(
        util.run_schedule(runner, util.schedule_tail("r3", reqs["r3"], 12))["r3"], ref["r3"],
        atol=3e-5, rtol=1e-4)
    d16 = str(tmp_path / "toy_scored_bf16")
    ninfer_amd.write_random_model(d16, toy.TOY_SCORED_CONFIG, 12, dtype="bfloat16", std=0.3)
    _, w16 = util.read_folder(d16)
    ref16 = toy.plain_forward_routed(w16, cfg, reqs["r3"])
    r16 = load_model(d16, EngineOptions(dtype="bfloat16", max_context=64, num_sequences=3,
                                        page_size=4, check_pages=True))
    got16 = util.run_schedule(r16, util.schedule_tail("r3", reqs["r3"], 12))["r3"]
    # Routing is discontinuous, so single rows have no bound in bfloat16. What is asked: the
    # typical row lies far closer to the plain model with this router than to the one whose
    # weights are not scaled.
    other = toy.plain_forward_routed(w16, dict(cfg, route_scale=1.0), reqs["r3"])
    err = (got16 - ref16).abs().max(-1).values
    wrong = (got16 - other).abs().max(-1).values
    assert float(err.median()) < float(wrong.median()) / 3
    assert float(err.median()) < 0.03 * float(ref16.abs().max())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_learned_positions_and_score_bias_on_the_gpu(tmp_path, dtype):
    """Positions without a rotation: learned absolute positions gathered in the embedding
    kernel and a distance-based bias in the attention kernels (heads of 64 and pages of 16: in
    bfloat16 the matrix-core prompt kernel and the split-context decode kernel), prompts in
    portions beside decoded tokens, the tail token by token."""
    import ninfer_amd
    from ninfer_amd import EngineOptions, load_model
    toy.register_routed()
    cfg = toy.TOY_BIASED_CONFIG
    d = str(tmp_path / "toy_biased")
    # (heads of 64 x 4 into a width of 64: std 0.2 keeps the logits at the size of the other toys',
    # for which the 32-bit bound below is made)
    ninfer_amd.write_random_model(d, cfg, 14, dtype=dtype, std=0.2)
    _, w = util.read_folder(d)
    runner = load_model(d, EngineOptions(dtype=dtype, max_context=160, num_sequences=3, page_size=16,
                                         check_pages=True))
    reqs = {f"r{i}": util.random_tokens(n, 83, 70 + i) for i, n in enumerate([7, 96, 15, 150])}
    ref = {k: toy.plain_forward_routed(w, cfg, v) for k, v in reqs.items()}
    got = util.run_schedule(runner, util.schedule_mixed(reqs, seed=8, max_live=3))
    tail = util.run_schedule(runner, util.schedule_tail("r3", reqs["r3"], 32))["r3"]
    if dtype == "float32":
        for k in reqs:
            torch.testing.assert_close(got[k], ref[k], atol=3e-5, rtol=1e-4)
        torch.testing.assert_close(tail, ref["r3"], atol=3e-5, rtol=1e-4)
    else:
        # (routing is discontinuous: the typical row is what is bounded in bfloat16)
        top = float(ref["r3"].abs().max())
        for rows in (got["r3"], tail, got["r1"]):
            want = ref["r3"] if rows.shape[0] == 150 else ref["r1"]
            err = (rows - want).abs().max(-1).values
            assert float(err.median()) < 0.03 * top
    with pytest.raises(ValueError, match="160 positions"):
        load_model(d, EngineOptions(dtype=dtype, max_context=176, num_sequences=1, page_size=16))


@pytest.mark.parametrize("dtype,graph", [("float32", False), ("bfloat16", False), ("bfloat16", True)])
def test_attention_layers_with_pages_of_other_sizes_on_the_gpu(tmp_path, dtype, graph):
    """A page size per layer (8, 32 and the engine's 16; heads of 64, so that the bfloat16 steps
    run the matrix-core kernels with each): three cache groups with block tables of their own,
    so few pages that they are used again, decoding also from a captured graph (whose tables
    have each group's full width)."""
    import ninfer_amd
    from ninfer_amd import EngineOptions, load_model
    toy.register_routed()
    cfg = toy.TOY_PAGES_CONFIG
    d = str(tmp_path / "toy_pages")
    ninfer_amd.write_random_model(d, cfg, 16, dtype=dtype, std=0.2)
    _, w = util.read_folder(d)
    runner = load_model(d, EngineOptions(dtype=dtype, max_context=160, num_sequences=3, page_size=16,
                                         num_pages=22, check_pages=True, poison_freed_pages=True,
                                         use_graph=graph))
    assert [(g.page_size, g.allocator.num_pages, g.max_pages) for g in runner.cache.groups] == \
        [(8, 44, 20), (32, 11, 5), (16, 22, 10)]
    reqs = {f"r{i}": util.random_tokens(n, 83, 90 + i) for i, n in enumerate([7, 96, 15, 150, 33])}
    ref = {k: toy.plain_forward_routed(w, cfg, v) for k, v in reqs.items()}
    got = util.run_schedule(runner, util.schedule_mixed(reqs, seed=5, max_live=3))
    tail = util.run_schedule(runner, util.schedule_tail("r3", reqs["r3"], 32))["r3"]
    if dtype == "float32":
        for k in reqs:
            torch.testing.assert_close(got[k], ref[k], atol=3e-5, rtol=1e-4)
        torch.testing.assert_close(tail, ref["r3"], atol=3e-5, rtol=1e-4)
    else:
        top = float(ref["r3"].abs().max())
        for rows in (got["r3"], tail, got["r1"]):
            assert torch.isfinite(rows).all()
            want = ref["r3"] if rows.shape[0] == 150 else ref["r1"]
            err = (rows - want).abs().max(-1).values
            assert float(err.median()) < 0.03 * top
    runner.cache.check()
    assert runner.cache.pages_reused() > 0
    assert bool(runner._graphs) == graph


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_normed_query_and_key_heads_on_the_gpu(tmp_path, dtype):
    """Query and key heads normed over their dims before the rotation, in the rotation's kernel
    (one wave per row and head), prompts in portions beside decoded tokens."""
    import ninfer_amd
    from ninfer_amd import EngineOptions, load_model
    toy.register_routed()
    cfg = toy.TOY_QK_NORM_CONFIG
    d = str(tmp_path / "toy_qk_norm")
    ninfer_amd.write_random_model(d, cfg, 15, dtype=dtype, std=0.3)
    _, w = util.read_folder(d)
    runner = load_model(d, EngineOptions(dtype=dtype, max_context=64, num_sequences=3, page_size=4,
                                         check_pages=True))
    reqs = {f"r{i}": util.random_tokens(n, 83, 80 + i) for i, n in enumerate([7, 26, 15, 33])}
    ref = {k: toy.plain_forward_routed(w, cfg, v) for k, v in reqs.items()}
    got = util.run_schedule(runner, util.schedule_mixed(reqs, seed=9, max_live=3))
    tail = util.run_schedule(runner, util.schedule_tail("r3", reqs["r3"], 12))["r3"]
    if dtype == "float32":
        for k in reqs:
            torch.testing.assert_close(got[k], ref[k], atol=3e-5, rtol=1e-4)
        torch.testing.assert_close(tail, ref["r3"], atol=3e-5, rtol=1e-4)
    else:
        # (one expert per token: a row that routes otherwise is far off, so the typical row is
        # what is bounded in bfloat16, against the model without the norm too)
        other = toy.plain_forward_routed(w, dict(cfg, qk_norm_eps=None), reqs["r3"])
        err = (tail - ref["r3"]).abs().max(-1).values
        wrong = (tail - other).abs().max(-1).values
        assert float(err.median()) < float(wrong.median()) / 3
        assert float(err.median()) < 0.03 * float(ref["r3"].abs().max())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_interleaved_pairs_on_the_gpu(tmp_path, dtype):
    """Neighbouring dims as rotation pairs (a partial rotation of 12 of 16 dims), chosen by
    the position encoding alone: the rotation kernel takes the pairing as a parameter."""
    import ninfer_amd
    from ninfer_amd import EngineOptions, load_model
    toy.register_routed()
    cfg = dict(toy.TOY_ROUTED_CONFIG, pairing="interleaved", rot_dim=12)
    d = str(tmp_path / "toy_interleaved")
    ninfer_amd.write_random_model(d, cfg, 10, dtype=dtype, std=0.3)
    _, w = util.read_folder(d)
    runner = load_model(d, EngineOptions(dtype=dtype, max_context=64, num_sequences=3, page_size=4,
                                         check_pages=True))
    reqs = {f"r{i}": util.random_tokens(n, 83, 50 + i) for i, n in enumerate([7, 26, 15, 33])}
    ref = {k: toy.plain_forward_routed(w, cfg, v) for k, v in reqs.items()}
    half = toy.plain_forward_routed(w, dict(cfg, pairing="half"), reqs["r1"])
    assert (half - ref["r1"]).abs().max() > 1e-3, "the pairing must matter"
    if dtype == "float32":
        got = util.run_schedule(runner, util.schedule_mixed(reqs, seed=6, max_live=3))
        for k in reqs:
            torch.testing.assert_close(got[k], ref[k], atol=3e-5, rtol=1e-4)
    else:
        # One expert per token: a row whose two best experts are nearly tied may go either way
        # in bfloat16, so single rows have no bound. What is asked: the typical row lies far
        # closer to the plain model with these pairs than to the one with the other pairs.
        got = util.run_schedule(runner, util.schedule_portions("r3", reqs["r3"], 2))["r3"]
        other = toy.plain_forward_routed(w, dict(cfg, pairing="half"), reqs["r3"])
        err = (got - ref["r3"]).abs().max(-1).values
        wrong = (got - other).abs().max(-1).values
        assert float(err.median()) < float(wrong.median()) / 3
        assert float(err.median()) < 0.03 * float(ref["r3"].abs().max())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_mixer_with_pools_of_its_own_on_the_gpu(tmp_path, dtype):
    """The third toy: a mixer with two paged pools of different widths and dtypes (the latent
    is 32-bit also in the bfloat16 engine), a window on one layer, freed pages poisoned."""
    import ninfer_amd
    from ninfer_amd import EngineOptions, load_model
    toy.register_latent()
    cfg = toy.TOY_LATENT_CONFIG
    d = str(tmp_path / "toy_latent")
    ninfer_amd.write_random_model(d, cfg, 12, dtype=dtype, std=0.2)
    _, w = util.read_folder(d)
    runner = load_model(d, EngineOptions(dtype=dtype, max_context=64, num_sequences=3, page_size=4,
                                         num_pages=26, poison_freed_pages=True, check_pages=True))
    pools = runner.cache.pools[0]
    assert pools["latent"].dtype == torch.float32 and pools["latent"].shape == (26, 4, 12)
    assert pools["pos_key"].dtype == runner.act_dtype and pools["pos_key"].shape == (26, 4, 6)
    reqs = {f"l{i}": util.random_tokens(n, 61, 70 + i) for i, n in enumerate([9, 30, 17, 41, 5])}
    ref = {k: toy.plain_forward_latent(w, cfg, v) for k, v in reqs.items()}
    # bfloat16 keeps three digits: the bound follows the size of the logits
    size = max(float(r.abs().max()) for r in ref.values())
    bound = dict(atol=3e-5, rtol=1e-4) if dtype == "float32" else dict(atol=0.03 * size, rtol=0.05)
    got = util.run_schedule(runner, util.schedule_mixed(reqs, seed=8, max_live=3))
    for k in reqs:
        assert torch.isfinite(got[k]).all()
        torch.testing.assert_close(got[k], ref[k], **bound)
    torch.testing.assert_close(
        util.run_schedule(runner, util.schedule_tail("l3", reqs["l3"], 7))["l3"], ref["l3"], **bound)
    runner.cache.check()
    assert runner.cache.pages_reused() > 0 and runner.cache.groups[1].window_freed > 0
    assert torch.isnan(pools["latent"]).any() and torch.isnan(pools["pos_key"]).any()


@pytest.mark.parametrize("plan", [[(0, None), (1, 0), (2, None)],
                                  [(0, None), (1, None), (1, None), (2, None)]])
def test_layer_plan_on_the_gpu(model_dirs, plan):
    from ninfer_amd import EngineOptions
    from ninfer_amd.config import read_config_json
    from ninfer_amd.engine import ModelRunner
    from ninfer_amd.loading import build_spec
    from ninfer_amd.models.spec import LayerCall
    from ninfer_amd.weights import CheckpointSource
    d = model_dirs["B"]["float32"]
    cfg, w = util.read_folder(d)
    _, spec = build_spec(read_config_json(d))
    spec.set_plan([LayerCall(l, c) for l, c in plan])
    runner = ModelRunner(spec, CheckpointSource(d),
                         EngineOptions(dtype="float32", max_context=64, num_sequences=2, page_size=8))
    toks = util.random_tokens(45, cfg["vocab_size"], 77)
    ref = plain_model.forward(w, cfg, toks, plan=plan)
    for sched in (util.schedule_whole("x", toks), util.schedule_portions("x", toks, 2)):
        torch.testing.assert_close(util.run_schedule(runner, sched)["x"], ref, atol=2e-5, rtol=1e-4)
