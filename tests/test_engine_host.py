"""The engine's host logic on the CPU: batch building, block tables, cache
manager, layer plan and state slots run end to end, with the plain twins of
the kernels (tests/plain_ops.py) in place of the HIP library, against the
plain implementation. The same replays run on the GPU with the real kernels in
test_engine_gpu.py."""
import pytest
import torch

import plain_model
import toy
import util
from conftest import TINY
from plain_ops import PlainOps


def runner_for(model_dir, page_size=8, num_pages=24, seqs=4, plan=None):
    from ninfer_amd import EngineOptions, load_model
    from ninfer_amd.models.spec import LayerCall
    opt = EngineOptions(dtype="float32", max_context=128, num_sequences=seqs, page_size=page_size,
                        num_pages=num_pages, device="cpu")
    if plan is None:
        return load_model(model_dir, opt, ops=PlainOps())
    # the order layers run in is data: rebuild the runner with another plan
    from ninfer_amd.config import read_config_json
    from ninfer_amd.engine import ModelRunner
    from ninfer_amd.loading import build_spec
    from ninfer_amd.weights import CheckpointSource
    _, spec = build_spec(read_config_json(model_dir))
    spec.set_plan([LayerCall(l, c) for l, c in plan])
    return ModelRunner(spec, CheckpointSource(model_dir), opt, ops=PlainOps())


@pytest.mark.parametrize("name", ["A", "B"])
def test_every_way_of_cutting_equals_the_plain_model(model_dirs, name):
    d = model_dirs[name]["float32"]
    cfg, w = util.read_folder(d)
    runner = runner_for(d)
    reqs = {f"r{i}": util.random_tokens(n, cfg["vocab_size"], 10 + i)
            for i, n in enumerate([5, 40, 33, 20, 47, 17])}
    ref = {k: plain_model.forward(w, cfg, v) for k, v in reqs.items()}
    for k, v in reqs.items():
        for sched in (util.schedule_whole(k, v), util.schedule_tail(k, v),
                      util.schedule_portions(k, v, 3)):
            torch.testing.assert_close(util.run_schedule(runner, sched)[k], ref[k],
                                       atol=2e-5, rtol=1e-4)
    got = util.run_schedule(runner, util.schedule_mixed(reqs, seed=5))
    for k in reqs:
        torch.testing.assert_close(got[k], ref[k], atol=2e-5, rtol=1e-4)
    runner.cache.check()
    assert runner.cache.pages_reused() > 0
    assert all(g.allocator.in_use == 0 for g in runner.cache.groups)
    if name == "B":
        assert [g.window for g in runner.cache.groups] == [None, 24]
        assert runner.cache.groups[1].window_freed > 0


def test_mixed_schedule_has_portions_beside_single_tokens():
    reqs = {f"r{i}": list(range(n)) for i, n in enumerate([5, 40, 33, 20, 47])}
    steps = util.schedule_mixed(reqs, seed=5)
    assert max(len(e) for e, _ in steps) == 4
    assert any(any(len(t) > 1 for _, t, _ in e) and any(len(t) == 1 for _, t, _ in e)
               for e, _ in steps)
    assert min(len(t) for e, _ in steps for _, t, _ in e) == 1
    fed = {k: sum(len(t) for e, _ in steps for r, t, _ in e if r == k) for k in reqs}
    assert fed == {k: len(v) for k, v in reqs.items()}


@pytest.mark.parametrize("plan", [[(0, None), (1, 0), (2, None)],
                                  [(0, None), (1, None), (1, None), (2, None)],
                                  [(2, None), (0, None)]])
def test_layer_plan_is_data(model_dirs, plan):
    """A layer named twice, a layer that reads another call's cache, layers in
    another order: the same parts, another list."""
    d = model_dirs["B"]["float32"]
    cfg, w = util.read_folder(d)
    runner = runner_for(d, plan=plan)
    toks = util.random_tokens(45, cfg["vocab_size"], 77)
    ref = plain_model.forward(w, cfg, toks, plan=plan)
    for sched in (util.schedule_whole("x", toks), util.schedule_portions("x", toks, 2),
                  util.schedule_tail("x", toks, 12)):
        torch.testing.assert_close(util.run_schedule(runner, sched)["x"], ref, atol=2e-5, rtol=1e-4)
    own_caches = sum(1 for _, src in plan if src is None)
    assert len(runner.cache.pools) == own_caches


def test_bad_plans_are_refused(model_dirs):
    with pytest.raises(ValueError, match="does not run before"):
        runner_for(model_dirs["B"]["float32"], plan=[(0, 1), (1, None)])
    with pytest.raises(ValueError, match="names layer 7"):
        runner_for(model_dirs["B"]["float32"], plan=[(7, None)])
    with pytest.raises(ValueError, match="no cache of its own"):
        runner_for(model_dirs["B"]["float32"], plan=[(0, None), (1, 0), (2, 1)])


def test_step_refuses_bad_batches(model_dirs):
    from ninfer_amd import Chunk
    from ninfer_amd.cache import OutOfPages
    runner = runner_for(model_dirs["A"]["float32"], num_pages=4)
    s = runner.open()
    with pytest.raises(ValueError, match="once in a step"):
        runner.step([Chunk(s, [1], []), Chunk(s, [2], [])])
    with pytest.raises(ValueError, match="token id"):
        runner.step([Chunk(s, [99999], [])])
    with pytest.raises(ValueError, match="at least one token"):
        runner.step([Chunk(s, [], [])])
    with pytest.raises(ValueError, match="wanted row"):
        runner.step([Chunk(s, [1, 2], [2])])
    with pytest.raises(OutOfPages):
        runner.step([Chunk(s, list(range(40)), [])])
    assert runner.cache.length(s) == 0 and runner.cache.pages_free(0) == 4
    assert runner.step([Chunk(s, [1, 2, 3], [])]) is None      # nothing wanted: no logits


def test_toy_mixer_with_state_of_its_own(tmp_path):
    """Registered, written, loaded and stepped through the framework's own entry
    points; its state lives in the request's slot, is carried across steps and
    is zeroed when a slot is used again."""
    import ninfer_amd
    toy.register()
    d = str(tmp_path / "toy")
    ninfer_amd.write_random_model(d, toy.TOY_CONFIG, 5, std=0.2)
    cfg, w = util.read_folder(d)
    runner = runner_for(d, seqs=3)
    assert runner.cache.state_floats == 2 * 40 and not runner.cache.pools
    reqs = {f"t{i}": util.random_tokens(n, 97, 60 + i) for i, n in enumerate([9, 21, 14, 30, 6])}
    ref = {k: toy.plain_forward(w, cfg, v) for k, v in reqs.items()}
    for k, v in reqs.items():
        for sched in (util.schedule_whole(k, v), util.schedule_tail(k, v, 5),
                      util.schedule_portions(k, v, 1)):
            torch.testing.assert_close(util.run_schedule(runner, sched)[k], ref[k],
                                       atol=2e-5, rtol=1e-4)
    got = util.run_schedule(runner, util.schedule_mixed(reqs, seed=3, max_live=3))
    for k in reqs:
        torch.testing.assert_close(got[k], ref[k], atol=2e-5, rtol=1e-4)


def test_toy_feed_forward_with_biases_and_another_activation(tmp_path):
    """The dense feed-forward with the tanh form of GELU as its gate's activation and a bias on
    each of its three products: parameters of the framework's part."""
    import ninfer_amd
    toy.register()
    cfg = toy.TOY_BIASED_MLP_CONFIG
    d = str(tmp_path / "toy_biased_mlp")
    ninfer_amd.write_random_model(d, cfg, 6, std=0.2)
    _, w = util.read_folder(d)
    assert w["layers.1.mlp.up_proj.bias"].shape == (56,) and w["layers.0.mlp.down_proj.bias"].shape == (40,)
    runner = runner_for(d, seqs=3)
    reqs = {f"t{i}": util.random_tokens(n, 97, 90 + i) for i, n in enumerate([9, 21, 14])}
    ref = {k: toy.plain_forward(w, cfg, v) for k, v in reqs.items()}
    assert (toy.plain_forward(w, dict(cfg, mlp_bias=False), reqs["t1"]) - ref["t1"]).abs().max() > 1e-3
    assert (toy.plain_forward(w, dict(cfg, hidden_act="silu"), reqs["t1"]) - ref["t1"]).abs().max() > 1e-3
    got = util.run_schedule(runner, util.schedule_mixed(reqs, seed=3, max_live=3))
    for k in reqs:
        torch.testing.assert_close(got[k], ref[k], atol=2e-5, rtol=1e-4)


def test_toy_routed_feed_forward_and_another_position_encoding(tmp_path):
    """A feed-forward with routing of its own (a router bias from the checkpoint,
    one expert per token) and a position encoding with other angles and a
    partial rotation, both defined in the tests, run through the framework's
    attention, cache, routing and grouped products, whole and in portions."""
    import ninfer_amd
    toy.register_routed()
    d = str(tmp_path / "toy_routed")
    ninfer_amd.write_random_model(d, toy.TOY_ROUTED_CONFIG, 9, std=0.3)
    cfg, w = util.read_folder(d)
    assert "layers.1.ff.router.bias" in w and "layers.0.ff.experts.4.down_proj.weight" in w
    runner = runner_for(d, seqs=3)
    assert len(runner.cache.pools) == 2          # one windowed cache per layer
    reqs = {f"r{i}": util.random_tokens(n, 83, 40 + i) for i, n in enumerate([7, 26, 15, 33])}
    ref = {k: toy.plain_forward_routed(w, cfg, v) for k, v in reqs.items()}
    for k, v in reqs.items():
        for sched in (util.schedule_whole(k, v), util.schedule_tail(k, v, 5),
                      util.schedule_portions(k, v, 2)):
            torch.testing.assert_close(util.run_schedule(runner, sched)[k], ref[k],
                                       atol=3e-5, rtol=1e-4)
    got = util.run_schedule(runner, util.schedule_mixed(reqs, seed=4, max_live=3))
    for k in reqs:
        torch.testing.assert_close(got[k], ref[k], atol=3e-5, rtol=1e-4)


def test_toy_router_with_other_scores(tmp_path):
    """A router of another kind (sigmoid scores, a bias of the checkpoint that decides the
    choice only, renormalised and scaled weights) built from the framework's router part by
    parameters alone."""
    import ninfer_amd
    toy.register_routed()
    d = str(tmp_path / "toy_scored")
    ninfer_amd.write_random_model(d, toy.TOY_SCORED_CONFIG, 12, std=0.3)
    cfg, w = util.read_folder(d)
    assert w["layers.1.ff.router.choice_bias"].shape == (6,)
    runner = runner_for(d, seqs=3)
    reqs = {f"r{i}": util.random_tokens(n, 83, 60 + i) for i, n in enumerate([7, 26, 15])}
    ref = {k: toy.plain_forward_routed(w, cfg, v) for k, v in reqs.items()}
    softmax_like = toy.plain_forward_routed(w, dict(cfg, route_scale=1.0), reqs["r1"])
    assert (softmax_like - ref["r1"]).abs().max() > 1e-3, "the scale must matter"
    ungrouped = toy.plain_forward_routed(w, dict(cfg, n_group=0), reqs["r1"])
    assert (ungrouped - ref["r1"]).abs().max() > 1e-3, "the groups must matter"
    got = util.run_schedule(runner, util.schedule_mixed(reqs, seed=5, max_live=3))
    for k in reqs:
        torch.testing.assert_close(got[k], ref[k], atol=3e-5, rtol=1e-4)


def test_toy_learned_positions_and_score_bias(tmp_path):
    """Positions without a rotation: a table of learned absolute positions gathered in the
    embedding, and a distance-based bias on the attention scores; both are parameters of the
    framework's parts. A context beyond the table's rows is refused when the engine is made."""
    import ninfer_amd
    from ninfer_amd import EngineOptions, load_model
    toy.register_routed()
    cfg = toy.TOY_BIASED_CONFIG
    d = str(tmp_path / "toy_biased")
    ninfer_amd.write_random_model(d, cfg, 14, std=0.3)
    _, w = util.read_folder(d)
    assert w["embed_positions.weight"].shape == (160, 64)
    runner = runner_for(d, seqs=3)
    reqs = {f"r{i}": util.random_tokens(n, 83, 70 + i) for i, n in enumerate([7, 26, 15])}
    ref = {k: toy.plain_forward_routed(w, cfg, v) for k, v in reqs.items()}
    w0 = dict(w, **{"embed_positions.weight": torch.zeros_like(w["embed_positions.weight"])})
    assert (toy.plain_forward_routed(w0, cfg, reqs["r1"]) - ref["r1"]).abs().max() > 1e-3, \
        "the learned positions must matter"
    got = util.run_schedule(runner, util.schedule_mixed(reqs, seed=7, max_live=3))
    for k in reqs:
        torch.testing.assert_close(got[k], ref[k], atol=3e-5, rtol=1e-4)
    with pytest.raises(ValueError, match="160 positions"):
        load_model(d, EngineOptions(dtype="float32", device="cpu", max_context=161, num_sequences=1,
                                    page_size=4), ops=PlainOps())


def test_attention_layers_with_pages_of_other_sizes(tmp_path):
    """The framework's attention part with a page size per layer (8, 32 and the engine's 16):
    three groups with block tables of their own, the same logits."""
    import ninfer_amd
    toy.register_routed()
    cfg = toy.TOY_PAGES_CONFIG
    d = str(tmp_path / "toy_pages")
    ninfer_amd.write_random_model(d, cfg, 16, std=0.3)
    _, w = util.read_folder(d)
    runner = runner_for(d, page_size=16, num_pages=12, seqs=3)
    assert [(g.page_size, g.allocator.num_pages) for g in runner.cache.groups] == \
        [(8, 24), (32, 6), (16, 12)]
    assert runner.cache.pools[1]["k"].shape == (6, 2, 32, 64)
    reqs = {f"r{i}": util.random_tokens(n, 83, 90 + i) for i, n in enumerate([7, 70, 15, 40, 33])}
    ref = {k: toy.plain_forward_routed(w, cfg, v) for k, v in reqs.items()}
    got = util.run_schedule(runner, util.schedule_mixed(reqs, seed=5, max_live=3))
    for k in reqs:
        torch.testing.assert_close(got[k], ref[k], atol=3e-5, rtol=1e-4)
    runner.cache.check()
    assert runner.cache.pages_reused() > 0


def test_toy_normed_query_and_key_heads(tmp_path):
    """Attention whose query and key heads are normed over their dims before they turn: a
    parameter of the attention part (two gain vectors of the checkpoint) and of the rotation's
    kernel."""
    import ninfer_amd
    toy.register_routed()
    cfg = toy.TOY_QK_NORM_CONFIG
    d = str(tmp_path / "toy_qk_norm")
    ninfer_amd.write_random_model(d, cfg, 15, std=0.3)
    _, w = util.read_folder(d)
    assert w["layers.0.attn.q_norm.weight"].shape == (16,)
    runner = runner_for(d, seqs=3)
    reqs = {f"r{i}": util.random_tokens(n, 83, 80 + i) for i, n in enumerate([7, 26, 15])}
    ref = {k: toy.plain_forward_routed(w, cfg, v) for k, v in reqs.items()}
    plain = toy.plain_forward_routed(w, dict(cfg, qk_norm_eps=None), reqs["r1"])
    assert (plain - ref["r1"]).abs().max() > 1e-3, "the heads' norm must matter"
    got = util.run_schedule(runner, util.schedule_mixed(reqs, seed=9, max_live=3))
    for k in reqs:
        torch.testing.assert_close(got[k], ref[k], atol=3e-5, rtol=1e-4)


def test_toy_interleaved_pairs(tmp_path):
    """The second toy with neighbouring dims as rotation pairs: the pairing is a property of
    the position encoding that attention hands to the rotation, nothing else changes."""
    import ninfer_amd
    toy.register_routed()
    cfg = dict(toy.TOY_ROUTED_CONFIG, pairing="interleaved", rot_dim=12)
    d = str(tmp_path / "toy_interleaved")
    ninfer_amd.write_random_model(d, cfg, 10, std=0.3)
    _, w = util.read_folder(d)
    runner = runner_for(d, seqs=3)
    reqs = {f"r{i}": util.random_tokens(n, 83, 50 + i) for i, n in enumerate([7, 26, 15])}
    ref = {k: toy.plain_forward_routed(w, cfg, v) for k, v in reqs.items()}
    half = toy.plain_forward_routed(w, dict(cfg, pairing="half"), reqs["r1"])
    assert (half - ref["r1"]).abs().max() > 1e-3, "the pairing must matter"
    got = util.run_schedule(runner, util.schedule_mixed(reqs, seed=6, max_live=3))
    for k in reqs:
        torch.testing.assert_close(got[k], ref[k], atol=3e-5, rtol=1e-4)


def test_toy_mixer_with_pools_of_its_own(tmp_path):
    """A mixer whose paged cache is two pools of different widths and dtypes (a 32-bit latent
    that is key and value at once, a short rotated key in the activation dtype), one layer
    with a window: the cache manager allocates, groups, frees and reuses its pages as it
    does attention's, and nothing of the framework is changed for it."""
    import ninfer_amd
    toy.register_latent()
    cfg = toy.TOY_LATENT_CONFIG
    d = str(tmp_path / "toy_latent")
    ninfer_amd.write_random_model(d, cfg, 12, std=0.3)
    _, w = util.read_folder(d)
    runner = runner_for(d, page_size=4, num_pages=26, seqs=3)
    pools = runner.cache.pools
    assert sorted(pools[0]) == ["latent", "pos_key"] and pools[0]["latent"].shape == (26, 4, 12)
    assert pools[1]["pos_key"].shape == (26, 4, 6)
    assert [g.window for g in runner.cache.groups] == [None, 9]
    assert runner.cache.kv_bytes_per_token(4) == 2 * (12 * 4 + 6 * 4)
    assert runner.cache.kv_bytes_per_token(2) == 2 * (12 * 4 + 6 * 2)   # the latent stays 32-bit
    reqs = {f"l{i}": util.random_tokens(n, 61, 70 + i) for i, n in enumerate([9, 30, 17, 41, 5])}
    ref = {k: toy.plain_forward_latent(w, cfg, v) for k, v in reqs.items()}
    for k, v in reqs.items():
        for sched in (util.schedule_whole(k, v), util.schedule_tail(k, v, 5),
                      util.schedule_portions(k, v, 1)):
            torch.testing.assert_close(util.run_schedule(runner, sched)[k], ref[k],
                                       atol=3e-5, rtol=1e-4)
    got = util.run_schedule(runner, util.schedule_mixed(reqs, seed=8, max_live=3))
    for k in reqs:
        torch.testing.assert_close(got[k], ref[k], atol=3e-5, rtol=1e-4)
    runner.cache.check()
    assert runner.cache.pages_reused() > 0 and runner.cache.groups[1].window_freed > 0


def test_toy_mixer_with_a_page_size_of_its_own(tmp_path):
    """A mixer may ask for pages of another size than the engine's: its layers form a group of
    their own with as many pages as hold the same number of tokens, their own block tables and
    their own giving back; the step function and the scheduler take each group's page size."""
    import ninfer_amd
    from ninfer_amd import Request, SamplingParams, Scheduler
    toy.register_latent()
    cfg = dict(toy.TOY_LATENT_CONFIG, windows=[None, 9, None], page_sizes=[None, 8, 2],
               num_hidden_layers=3)
    d = str(tmp_path / "toy_latent_pages")
    ninfer_amd.write_random_model(d, cfg, 12, std=0.3)
    _, w = util.read_folder(d)
    runner = runner_for(d, page_size=4, num_pages=26, seqs=3)
    cache = runner.cache
    assert [(g.window, g.page_size, g.allocator.num_pages, g.max_pages) for g in cache.groups] == \
        [(None, 4, 26, 32), (9, 8, 13, 16), (None, 2, 52, 64)]
    assert cache.pools[1]["latent"].shape == (13, 8, 12) and cache.pools[2]["pos_key"].shape == (52, 2, 6)
    reqs = {f"l{i}": util.random_tokens(n, 61, 70 + i) for i, n in enumerate([9, 30, 17, 41, 5])}
    ref = {k: toy.plain_forward_latent(w, cfg, v) for k, v in reqs.items()}
    for k, v in reqs.items():
        for sched in (util.schedule_whole(k, v), util.schedule_tail(k, v, 5),
                      util.schedule_portions(k, v, 1)):
            torch.testing.assert_close(util.run_schedule(runner, sched)[k], ref[k],
                                       atol=3e-5, rtol=1e-4)
    got = util.run_schedule(runner, util.schedule_mixed(reqs, seed=8, max_live=3))
    for k in reqs:
        torch.testing.assert_close(got[k], ref[k], atol=3e-5, rtol=1e-4)
    cache.check()
    assert cache.pages_reused() > 0 and cache.groups[1].window_freed > 0
    # the scheduler plans with every group's page size (here the pages of 2 tokens run out first)
    sched = Scheduler(runner, None, max_batch_tokens=16, max_seqs=3)
    assert sched._fits_alone(100) and not sched._fits_alone(105)   # 52 pages of 2 tokens


def test_page_checks_name_a_table_that_the_kernels_could_not_trust(model_dirs):
    """The debugging option checks every step's block tables on the host before anything is
    launched: a page number outside the pool, a position without a held page, a page in two
    requests' tables."""
    from ninfer_amd import Chunk, EngineOptions, load_model
    opt = EngineOptions(dtype="float32", max_context=64, num_sequences=3, page_size=4,
                        num_pages=12, device="cpu", check_pages=True)
    runner = load_model(model_dirs["B"]["float32"], opt, ops=PlainOps())
    a, b = runner.open(), runner.open()
    runner.step([Chunk(a, list(range(9)), []), Chunk(b, list(range(5)), [])])
    g = runner.cache.groups[0]
    keep = g.rows[a, 1]
    g.rows[a, 1] = 99
    with pytest.raises(RuntimeError, match="outside"):
        runner.step([Chunk(a, [1], [0])])
    g.rows[a, 1] = -1
    with pytest.raises(RuntimeError, match="not held"):
        runner.step([Chunk(a, [1], [0])])
    g.rows[a, 1] = g.rows[b, 0]
    with pytest.raises(RuntimeError, match="slots"):
        runner.step([Chunk(a, [1], []), Chunk(b, [1], [])])
    g.rows[a, 1] = keep
    assert runner.step([Chunk(a, [1], [0]), Chunk(b, [2], [0])]).shape[0] == 2


def test_cache_sized_in_bytes(model_dirs):
    from ninfer_amd import EngineOptions, load_model
    # A: two layers of 2 kv heads x 16, keys and values, 32-bit: 2 * 2 * 2 * 16 * 4 = 512 bytes a token
    opt = EngineOptions(dtype="float32", max_context=64, num_sequences=2, page_size=8,
                        kv_bytes=512 * 8 * 10 + 100, device="cpu")
    runner = load_model(model_dirs["A"]["float32"], opt, ops=PlainOps())
    assert runner.cache.kv_bytes_per_token(4) == 512 and runner.cache.pages_total(0) == 10
    with pytest.raises(ValueError, match="not both"):
        EngineOptions(num_pages=4, kv_bytes=1 << 20).validate()
    with pytest.raises(ValueError, match="holds no page"):
        load_model(model_dirs["A"]["float32"],
                   EngineOptions(dtype="float32", kv_bytes=100, device="cpu"), ops=PlainOps())


def test_a_page_size_the_fast_attention_kernels_do_not_take_is_said(recwarn):
    """bfloat16 with pages that are no power of two, or of more than 64 tokens, runs on the plain
    attention kernel: right and slow, and the options say so; 32-bit runs it anyway."""
    import warnings
    from ninfer_amd import EngineOptions
    for ps in (4, 16, 64):
        EngineOptions(dtype="bfloat16", page_size=ps).validate()
    EngineOptions(dtype="float32", page_size=48).validate()
    assert not [w for w in recwarn.list if "page_size" in str(w.message)]
    for ps in (48, 128, 24, 2):
        with pytest.warns(UserWarning, match=f"page_size {ps}.*plain attention kernel"):
            EngineOptions(dtype="bfloat16", page_size=ps).validate()
    # ... and so of a page size that a mixer asks for itself
    opt = EngineOptions(dtype="bfloat16", page_size=16)
    opt.warn_of_slow_pages(32)
    assert not [w for w in recwarn.list if "page_size 32" in str(w.message)]
    with pytest.warns(UserWarning, match="page_size 24.*plain attention kernel"):
        opt.warn_of_slow_pages(24)
    with pytest.raises(ValueError, match="max_graphs"):
        EngineOptions(max_graphs=0).validate()


def test_weights_can_be_read_back_by_name(model_dirs):
    """What the engine holds under a checkpoint name, fused and stacked tensors included,
    is what the folder holds."""
    d = model_dirs["B"]["float32"]
    _, w = util.read_folder(d)
    runner = runner_for(d)
    assert set(runner.tensor_names()) == set(w) 
    for name, t in w.items():
        assert torch.equal(runner.tensor(name).float().cpu().reshape(t.shape), t), name
    with pytest.raises(KeyError):
        runner.tensor("no.such.weight")
