"""The scheduler's decisions, on the CPU: the engine's host logic runs with the
plain twins of the kernels (tests/plain_ops.py) in place of the HIP library."""
import random

import pytest
import torch

import plain_model
import util
from conftest import TINY
from plain_ops import PlainOps


@pytest.fixture(scope="module")
def setup(model_dirs):
    cfg, w = util.read_folder(model_dirs["A"]["float32"])
    return model_dirs["A"]["float32"], cfg, w


def make(setup, num_pages, page_size=4, chunk=16, seqs=4, max_context=96):
    from ninfer_amd import EngineOptions, Sampler, Scheduler, load_model
    opt = EngineOptions(dtype="float32", max_context=max_context, prefill_chunk=chunk,
                        num_sequences=seqs, page_size=page_size, num_pages=num_pages, device="cpu")
    runner = load_model(setup[0], opt, ops=PlainOps())
    return runner, Scheduler(runner, Sampler(PlainOps(), runner.device))


class Spy:
    """Wraps a runner's step to record the shape of every batch."""

    def __init__(self, runner):
        self.runner, self.batches = runner, []
        self._step = runner.step
        runner.step = self.step

    def step(self, chunks):
        self.batches.append([(c.slot, len(c.tokens), list(c.want)) for c in chunks])
        return self._step(chunks)


def requests(cfg, lens, max_new, **kw):
    from ninfer_amd import Request, SamplingParams
    params = SamplingParams(max_new_tokens=max_new, **kw)
    return [Request(f"q{i}", util.random_tokens(n, cfg["vocab_size"], 50 + i), params)
            for i, n in enumerate(lens)]


def test_greedy_matches_plain_and_budgets_hold(setup):
    _, cfg, w = setup
    runner, sched = make(setup, num_pages=200)
    spy = Spy(runner)
    reqs = requests(cfg, [5, 11, 17, 30, 3, 23], 8, temperature=0.0, top_k=0, top_p=1.0,
                    repetition_penalty=1.0)
    for r in reqs:
        sched.add(r)
    sched.run()
    for r in reqs:
        assert r.status == "finished" and len(r.output) == 8
        assert r.output == plain_model.greedy_generate(w, cfg, r.prompt, 8)
    for b in spy.batches:
        assert sum(n for _, n, _ in b) <= 16 and len(b) <= 4
        assert len({s for s, _, _ in b}) == len(b)
    # prompts longer than the budget were cut; some steps mix portions and decode tokens
    assert any(len(b) > 1 and any(n > 1 for _, n, _ in b) and any(n == 1 for _, n, _ in b)
               for b in spy.batches)
    runner.cache.check()
    assert all(g.allocator.in_use == 0 for g in runner.cache.groups)
    assert runner.cache.free_slots == 4


def test_preemption_gives_the_same_tokens(setup):
    _, cfg, w = setup
    lens = [20, 18, 22, 16]
    runner, sched = make(setup, num_pages=200)
    ref = requests(cfg, lens, 12, temperature=0.8, top_k=20, top_p=0.9, seed=77)
    for r in ref:
        sched.add(r)
    sched.run()
    # 22 pages of 4 tokens cannot hold four requests of ~30 tokens: some are preempted
    runner2, sched2 = make(setup, num_pages=22)
    again = requests(cfg, lens, 12, temperature=0.8, top_k=20, top_p=0.9, seed=77)
    for r in again:
        sched2.add(r)
    sched2.run()
    assert sched2.preemptions > 0
    for a, b in zip(ref, again):
        assert b.status == "finished" and a.output == b.output
    runner2.cache.check()
    assert all(g.allocator.in_use == 0 for g in runner2.cache.groups)


def test_request_that_cannot_fit_fails_alone(setup):
    _, cfg, _ = setup
    runner, sched = make(setup, num_pages=6)       # 24 tokens of cache
    big, small = requests(cfg, [40, 6], 4, temperature=0.0)
    sched.add(big)
    sched.add(small)
    sched.run()
    assert big.status == "failed" and "fit" in big.error
    assert small.status == "finished" and len(small.output) == 4
    assert all(g.allocator.in_use == 0 for g in runner.cache.groups)
    # a request that grows beyond the pool while decoding, alone, fails too
    runner, sched = make(setup, num_pages=6)
    (grow,) = requests(cfg, [20], 30, temperature=0.0)
    sched.add(grow)
    sched.run()
    assert grow.status == "failed" and len(grow.output) > 0
    assert all(g.allocator.in_use == 0 for g in runner.cache.groups)


def test_reference_rule_prompt_plus_new_tokens(setup):
    _, cfg, _ = setup
    runner, sched = make(setup, num_pages=200, max_context=32)
    (r,) = requests(cfg, [30], 8, temperature=0.0)
    sched.add(r)
    assert r.status == "failed" and "max_context" in r.error


def test_stop_token_ends_a_request(setup):
    _, cfg, w = setup
    runner, sched = make(setup, num_pages=200)
    (r,) = requests(cfg, [9], 10, temperature=0.0)
    full = plain_model.greedy_generate(w, cfg, r.prompt, 10)
    r.stop_ids = [full[4]]
    sched.add(r)
    sched.run()
    assert r.status == "finished" and r.output == full[:full.index(full[4])]


def test_seeded_sampling_does_not_depend_on_the_crowd(setup):
    _, cfg, _ = setup
    lens = [7, 13, 9]
    outs = []
    for crowd in (False, True):
        runner, sched = make(setup, num_pages=200)
        reqs = requests(cfg, lens if crowd else lens[:1], 10, temperature=1.0, top_k=0, top_p=1.0,
                        repetition_penalty=1.0, seed=5)
        for r in reqs:
            sched.add(r)
        sched.run()
        outs.append(reqs[0].output)
    assert outs[0] == outs[1]
    # and another seed gives another continuation
    runner, sched = make(setup, num_pages=200)
    (r,) = requests(cfg, lens[:1], 10, temperature=1.0, top_k=0, top_p=1.0,
                    repetition_penalty=1.0, seed=6)
    sched.add(r)
    sched.run()
    assert r.output != outs[0]


def test_random_arrivals_never_leak(setup):
    _, cfg, _ = setup
    rng = random.Random(3)
    runner, sched = make(setup, num_pages=40, chunk=12, seqs=3)
    pending = requests(cfg, [rng.randrange(2, 30) for _ in range(14)], 5, temperature=0.0)
    done = 0
    while pending or sched.has_work():
        while pending and rng.random() < 0.4:
            sched.add(pending.pop())
        if sched.has_work():
            done += len(sched.step())
            runner.cache.check()
    assert done == 14 and all(r.status == "finished" for r in sched.finished)
    assert all(g.allocator.in_use == 0 for g in runner.cache.groups)


def test_next_tokens_spans_prompt_and_output():
    from ninfer_amd import Request
    r = Request(id="a", prompt=[1, 2, 3, 4], output=[9, 8, 7])
    for cached in range(7):
        for n in range(1, 8 - cached):
            r.cached = cached
            assert r.next_tokens(n) == r.tokens[cached:cached + n]


def test_history_counts_like_a_counter():
    """The sampler's history (distinct tokens and counts as growing arrays) against
    collections.Counter, from a prompt and from nothing, beyond its first capacity."""
    import random
    from collections import Counter
    from ninfer_amd.sampling.sampler import History
    rng = random.Random(3)
    toks = [rng.randrange(400) for _ in range(1500)]
    for start in (0, 100):
        h = History(toks[:start])
        for t in toks[start:]:
            h.add(t)
        a, n = h.arrays()
        assert dict(zip(a.tolist(), n.tolist())) == dict(Counter(toks))
        assert len(h) == len(set(toks)) and h.count(toks[0]) == Counter(toks)[toks[0]]
        assert h.count(100000) == 0


def test_an_older_request_is_never_given_back_for_a_newer_one(setup):
    """An old request with a long prompt is still being fed in portions when a newer, short
    one is already decoding and the pool runs dry: the newer one waits or is preempted, the
    older one keeps its pages (it would have to recompute all its portions)."""
    _, cfg, w = setup
    runner, sched = make(setup, num_pages=14, chunk=8, max_context=96)   # 56 tokens of cache
    old, new = requests(cfg, [44, 6], 6, temperature=0.0, repetition_penalty=1.0)
    sched.add(old)
    sched.add(new)
    steps = 0
    while sched.has_work():
        sched.step()
        steps += 1
        assert old.preemptions == 0
        assert steps < 200
    assert old.status == "finished" and new.status == "finished"
    assert old.output == plain_model.greedy_generate(w, cfg, old.prompt, 6)
    assert new.output == plain_model.greedy_generate(w, cfg, new.prompt, 6)
    assert new.preemptions > 0, "the pool was meant to run dry while the old prompt was fed"
    runner.cache.check()
    assert all(g.allocator.in_use == 0 for g in runner.cache.groups)


def test_a_windowed_group_admits_what_its_window_can_serve(model_dirs):
    """All layers of this model see a window of 8 keys. Eleven pages of 4 tokens cannot hold
    the 60 tokens of the request, but they hold the window and one step's portion, and pages
    the window has passed come back after every step: the request runs, and its tokens are
    those of the plain model."""
    import json
    import os
    import ninfer_amd
    from ninfer_amd import EngineOptions, Request, SamplingParams, Sampler, Scheduler, load_model
    cfg = dict(TINY["B"][0], max_window_layers=0, sliding_window=8)
    d = os.path.join(os.path.dirname(model_dirs["B"]["float32"]), "windows_only")
    ninfer_amd.write_random_model(d, cfg, 5, std=0.1)
    raw, w = util.read_folder(d)
    opt = EngineOptions(dtype="float32", max_context=96, prefill_chunk=16, num_sequences=2,
                        page_size=4, num_pages=11, device="cpu", check_pages=True)
    runner = load_model(d, opt, ops=PlainOps())
    assert [g.window for g in runner.cache.groups] == [8]
    sched = Scheduler(runner, Sampler(PlainOps(), runner.device))
    req = Request("long", util.random_tokens(52, cfg["vocab_size"], 3),
                  SamplingParams.greedy(8))
    sched.add(req)
    sched.run()
    assert req.status == "finished", req.error
    assert req.output == plain_model.greedy_generate(w, raw, req.prompt, 8)
    assert runner.cache.groups[0].window_freed > 0
    # The boundary: a step of 16 tokens touches the 7 keys before its first row and its own 16
    # positions, 23 in all, which lie in at most ceil(23 / 4) + 1 = 7 pages. With exactly 7
    # the request runs (every step's tables checked); with 6 it is refused at admission.
    opt.num_pages = 7
    runner = load_model(d, opt, ops=PlainOps())
    sched = Scheduler(runner, Sampler(PlainOps(), runner.device))
    req3 = Request("long", list(req.prompt), SamplingParams.greedy(8))
    sched.add(req3)
    sched.run()
    assert req3.status == "finished", req3.error
    assert req3.output == req.output and req3.preemptions == 0
    for pages in (6, 5):
        opt.num_pages = pages
        runner = load_model(d, opt, ops=PlainOps())
        sched = Scheduler(runner, Sampler(PlainOps(), runner.device))
        req2 = Request("long", list(req.prompt), SamplingParams.greedy(8))
        sched.add(req2)
        sched.run()
        assert req2.status == "failed" and "fit" in req2.error


def test_groups_with_pages_of_other_sizes_under_the_scheduler(tmp_path):
    """Layers with pages of 8, 32 and 16 tokens (three cache groups): the scheduler counts
    every group's pages in that group's size, gives requests back when any group runs out,
    and the tokens are those of a run with room for everything."""
    import ninfer_amd
    import toy
    from ninfer_amd import EngineOptions, Request, SamplingParams, Sampler, Scheduler, load_model
    toy.register_routed()
    cfg = toy.TOY_PAGES_CONFIG
    d = str(tmp_path / "toy_pages")
    ninfer_amd.write_random_model(d, cfg, 16, std=0.3)

    def run(num_pages):
        opt = EngineOptions(dtype="float32", max_context=96, prefill_chunk=16, num_sequences=4,
                            page_size=16, num_pages=num_pages, device="cpu", check_pages=True)
        runner = load_model(d, opt, ops=PlainOps())
        sched = Scheduler(runner, Sampler(PlainOps(), runner.device))
        params = SamplingParams(max_new_tokens=12, temperature=0.8, top_k=20, top_p=0.9, seed=5)
        reqs = [Request(f"q{i}", util.random_tokens(n, 83, 60 + i), params)
                for i, n in enumerate([30, 28, 25, 21])]
        for r in reqs:
            sched.add(r)
        sched.run()
        runner.cache.check()
        assert all(g.allocator.in_use == 0 for g in runner.cache.groups)
        return runner, sched, reqs

    _, roomy, ref = run(64)
    assert roomy.preemptions == 0
    # 9 pages of 16 tokens, hence 18 of 8 and 4 of 32: the four prompts take a page of 32 each
    # and all are admitted; grown past 32 tokens each needs a second one, and there is none
    runner, tight, again = run(9)
    assert [(g.page_size, g.allocator.num_pages) for g in runner.cache.groups] == \
        [(8, 18), (32, 4), (16, 9)]
    assert tight.preemptions > 0
    for a, b in zip(ref, again):
        assert b.status == "finished" and a.output == b.output
    # a request that needs more pages of 32 than there are (3 of 2) fails alone
    runner, sched, _ = run(4)
    big = Request("big", util.random_tokens(70, 83, 1), SamplingParams.greedy(10))
    sched.add(big)
    sched.run()
    assert big.status == "failed" and "fit" in big.error
