"""Pins of the plain implementation beside the reference's text: special
cases that reduce to a library routine, and invariants, each chosen so that a
plausible mistake (a wrong sign or pairing, a norm in the wrong place, eps
outside the root, the wrong head sharing a kv head) fails it. The reference
ships no test vectors (it has no tests), so none are held here."""
import math

import pytest
import torch
import torch.nn.functional as F

import plain_model as pm
from conftest import CONFIG_A, CONFIG_B


def randn(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


# ---- RMSNorm ---------------------------------------------------------------
def test_rmsnorm_unit_gain_is_x_over_rms():
    x = randn(5, 48)
    ref = x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6)
    torch.testing.assert_close(pm.rms_norm(x, torch.ones(48), 1e-6), ref)


def test_rmsnorm_output_rms_is_one_and_scale_free():
    x = randn(4, 64, seed=1)
    y = pm.rms_norm(x, torch.ones(64), 1e-12)
    torch.testing.assert_close(y.pow(2).mean(-1), torch.ones(4))
    torch.testing.assert_close(pm.rms_norm(7.5 * x, torch.ones(64), 1e-12), y)


def test_rmsnorm_eps_is_inside_the_root():
    x = torch.full((1, 16), 1e-4)
    eps = 1e-2   # x^2 << eps: y ~ x / sqrt(eps); eps outside the root would give ~ x / (|x| + eps)
    y = pm.rms_norm(x, torch.ones(16), eps)
    torch.testing.assert_close(y, x / math.sqrt(eps + 1e-8))
    assert torch.equal(pm.rms_norm(torch.zeros(2, 8), torch.ones(8), 1e-6), torch.zeros(2, 8))


def test_rmsnorm_gain_multiplies_after_normalisation():
    x, w = randn(3, 32, seed=2), randn(32, seed=3)
    torch.testing.assert_close(pm.rms_norm(x, w, 1e-6), pm.rms_norm(x, torch.ones(32), 1e-6) * w)


# ---- rotary ------------------------------------------------------------------
def test_rope_position_zero_is_identity_and_norms_are_kept():
    x = randn(6, 3, 32, seed=4)
    assert torch.equal(pm.apply_rope(x, torch.zeros(6, dtype=torch.long), 1e4), x)
    y = pm.apply_rope(x, torch.arange(6) * 37, 1e4)
    half = 16
    torch.testing.assert_close(y[..., :half] ** 2 + y[..., half:] ** 2,
                               x[..., :half] ** 2 + x[..., half:] ** 2)


def test_rope_pairs_i_with_i_plus_half_and_turns_the_right_way():
    d = 16
    x = torch.zeros(1, 1, d)
    x[0, 0, 0] = 1.0
    y = pm.apply_rope(x, torch.tensor([1]), 1e4)   # f_0 = 1: angle of 1 radian
    expect = torch.zeros(d)
    expect[0], expect[d // 2] = math.cos(1.0), math.sin(1.0)   # into x_{D/2}, not x_1; + sin
    torch.testing.assert_close(y[0, 0], expect)


def test_rope_frequencies_are_geometric():
    f = pm.rope_inv_freq(32, 1e6)
    assert f[0] == 1.0 and f.shape == (16,)
    torch.testing.assert_close(f[1:] / f[:-1], torch.full((15,), 1e6 ** (-2 / 32)))


def test_rope_scores_depend_on_distance_only():
    q, k = randn(1, 1, 32, seed=5), randn(1, 1, 32, seed=6)
    def score(m, n):
        return (pm.apply_rope(q, torch.tensor([m]), 1e4) *
                pm.apply_rope(k, torch.tensor([n]), 1e4)).sum()
    torch.testing.assert_close(score(9, 4), score(105, 100), atol=1e-4, rtol=1e-4)
    assert abs(score(9, 4) - score(9, 5)) > 1e-3


# ---- attention ---------------------------------------------------------------
def test_attention_equals_library_sdpa_with_repeated_kv_heads():
    t, hq, hkv, d = 9, 6, 2, 16
    q, k, v = randn(t, hq, d, seed=7), randn(t, hkv, d, seed=8), randn(t, hkv, d, seed=9)
    pos = torch.arange(t)
    for window in (None, 4):
        mask = pm.visibility(pos, pos, window)
        ref = F.scaled_dot_product_attention(
            q.transpose(0, 1), k.repeat_interleave(hq // hkv, 1).transpose(0, 1),
            v.repeat_interleave(hq // hkv, 1).transpose(0, 1), attn_mask=mask).transpose(0, 1)
        torch.testing.assert_close(pm.attention_core(q, k, v, pos, pos, window), ref,
                                   atol=1e-5, rtol=1e-5)


def test_attention_single_visible_key_and_equal_scores():
    t, d = 5, 8
    q, v = randn(t, 2, d, seed=10), randn(t, 1, d, seed=11)
    pos = torch.arange(t)
    out = pm.attention_core(q, randn(t, 1, d, seed=12), v, pos, pos, 1)   # window 1: only itself
    torch.testing.assert_close(out, v.expand(t, 2, d))
    out = pm.attention_core(q, torch.zeros(t, 1, d), v, pos, pos, None)   # equal scores: mean
    torch.testing.assert_close(out[3, 0], v[:4, 0].mean(0))


def test_attention_window_covers_exactly_window_keys():
    pos = torch.arange(10)
    vis = pm.visibility(pos, pos, 3)
    assert vis[9].nonzero().flatten().tolist() == [7, 8, 9]
    assert torch.equal(pm.visibility(pos, pos, 10), pm.visibility(pos, pos, None))


def test_attention_scale_is_one_over_sqrt_d():
    t, d = 4, 16
    q, k, v = randn(t, 1, d, seed=13), randn(t, 1, d, seed=14), randn(t, 1, d, seed=15)
    pos = torch.arange(t)
    s = (q[:, 0] @ k[:, 0].T) / math.sqrt(d)
    s = s.masked_fill(~pm.visibility(pos, pos, None), float("-inf"))
    torch.testing.assert_close(pm.attention_core(q, k, v, pos, pos, None)[:, 0],
                               torch.softmax(s, -1) @ v[:, 0])


def test_attention_score_slopes_are_a_library_mask_of_distances():
    """A distance-based bias: library attention with the float mask slope_h * (j - i); slope 0
    is no bias; only distances count (all positions shifted: the same); a steep slope leaves a
    row its own key (a wrong sign would leave it the farthest)."""
    t, hq, hkv, d = 9, 4, 2, 16
    q, k, v = randn(t, hq, d, seed=41), randn(t, hkv, d, seed=42), randn(t, hkv, d, seed=43)
    pos = torch.arange(t)
    slopes = [0.5, 0.25, 0.0, 2.0]
    vis = pm.visibility(pos, pos, None)
    dist = (pos[None, :] - pos[:, None]).float()
    mask = torch.stack([s * dist for s in slopes]).masked_fill(~vis, float("-inf"))
    ref = F.scaled_dot_product_attention(
        q.transpose(0, 1), k.repeat_interleave(2, 1).transpose(0, 1),
        v.repeat_interleave(2, 1).transpose(0, 1), attn_mask=mask).transpose(0, 1)
    got = pm.attention_core(q, k, v, pos, pos, None, slopes)
    torch.testing.assert_close(got, ref, atol=1e-5, rtol=1e-5)
    plain = pm.attention_core(q, k, v, pos, pos, None)
    torch.testing.assert_close(got[:, 2], plain[:, 2])
    assert (got[:, 0] - plain[:, 0]).abs().max() > 1e-2
    torch.testing.assert_close(pm.attention_core(q, k, v, pos + 70, pos + 70, None, slopes), got)
    steep = pm.attention_core(q, k, v, pos, pos, None, [200.0] * hq)
    torch.testing.assert_close(steep, v.repeat_interleave(2, 1))


# ---- router and experts --------------------------------------------------------
def test_router_equals_library_softmax_topk():
    x, wr = randn(7, 24, seed=16), randn(10, 24, seed=17)
    ids, wts = pm.router(x, wr, 3, False)
    p = torch.softmax(x @ wr.T, -1)
    top = torch.topk(p, 3, dim=-1)
    assert torch.equal(ids, top.indices)
    torch.testing.assert_close(wts, top.values)
    assert (wts.sum(-1) < 1).all()
    _, wn = pm.router(x, wr, 3, True)
    torch.testing.assert_close(wn.sum(-1), torch.ones(7))
    _, wall = pm.router(x, wr, 10, True)     # k = E and renormalised: weights are p
    torch.testing.assert_close(wall.sort(-1).values, p.sort(-1).values)


def test_router_ties_go_to_the_lower_index():
    ids, _ = pm.router(torch.ones(1, 4), torch.zeros(6, 4), 2, False)
    assert ids.tolist() == [[0, 1]]


def _moe_weights(e, h, inner, same=False, seed=20):
    w = {}
    for i in range(e):
        s = seed if same else seed + i
        w[f"m.experts.{i}.gate_proj.weight"] = randn(inner, h, seed=s, scale=0.3)
        w[f"m.experts.{i}.up_proj.weight"] = randn(inner, h, seed=s + 100, scale=0.3)
        w[f"m.experts.{i}.down_proj.weight"] = randn(h, inner, seed=s + 200, scale=0.3)
    return w


def test_identical_experts_renormalised_equal_one_dense_mlp():
    h, inner, e = 16, 24, 5
    w = _moe_weights(e, h, inner, same=True)
    x = randn(6, h, seed=30)
    ids, wts = pm.router(x, randn(e, h, seed=31), 3, True)
    dense = pm.swiglu_mlp(x, w["m.experts.0.gate_proj.weight"], w["m.experts.0.up_proj.weight"],
                          w["m.experts.0.down_proj.weight"])
    torch.testing.assert_close(pm.routed_experts(x, ids, wts, w, "m."), dense, atol=1e-5, rtol=1e-5)


def test_expert_permutation_leaves_the_output_unchanged():
    h, inner, e = 16, 24, 4
    w = _moe_weights(e, h, inner)
    wr = randn(e, h, seed=32)
    x = randn(5, h, seed=33)
    ids, wts = pm.router(x, wr, 2, False)
    y = pm.routed_experts(x, ids, wts, w, "m.")
    perm = [2, 0, 3, 1]
    w2 = {}
    for new, old in enumerate(perm):
        for name in ("gate_proj", "up_proj", "down_proj"):
            w2[f"m.experts.{new}.{name}.weight"] = w[f"m.experts.{old}.{name}.weight"]
    ids2, wts2 = pm.router(x, wr[perm], 2, False)
    torch.testing.assert_close(pm.routed_experts(x, ids2, wts2, w2, "m."), y)


def test_swiglu_uses_library_silu():
    x = randn(3, 8, seed=34)
    wg, wu, wd = randn(12, 8, seed=35), randn(12, 8, seed=36), randn(8, 12, seed=37)
    torch.testing.assert_close(pm.swiglu_mlp(x, wg, wu, wd), (F.silu(x @ wg.T) * (x @ wu.T)) @ wd.T)


def test_gelu_gate_uses_library_gelu():
    """`hidden_act` = 'gelu_pytorch_tanh': the library's tanh form (the erf form differs from
    it by up to 5e-4 at these inputs, which the bound would not let through)."""
    x = randn(5, 8, seed=134) * 2
    wg, wu, wd = randn(12, 8, seed=135), randn(12, 8, seed=136), randn(8, 12, seed=137)
    want = (F.gelu(x @ wg.T, approximate="tanh") * (x @ wu.T)) @ wd.T
    torch.testing.assert_close(pm.swiglu_mlp(x, wg, wu, wd, "gelu_pytorch_tanh"), want)
    g = torch.linspace(-4, 4, 101)
    torch.testing.assert_close(pm.gate_activation(g, "gelu_pytorch_tanh"), F.gelu(g, approximate="tanh"),
                               atol=2e-6, rtol=1e-6)
    assert (pm.gate_activation(g, "gelu_pytorch_tanh") - F.gelu(g)).abs().max() > 1e-4
    with pytest.raises(ValueError):
        pm.gate_activation(g, "relu")


def test_shared_expert_gate_zero_is_one_half():
    h, inner = 8, 12
    w = {"m.shared_expert.gate_proj.weight": randn(inner, h, seed=38),
         "m.shared_expert.up_proj.weight": randn(inner, h, seed=39),
         "m.shared_expert.down_proj.weight": randn(h, inner, seed=40),
         "m.shared_expert_gate.weight": torch.zeros(1, h)}
    x = randn(4, h, seed=41)
    s = pm.swiglu_mlp(x, w["m.shared_expert.gate_proj.weight"], w["m.shared_expert.up_proj.weight"],
                      w["m.shared_expert.down_proj.weight"])
    torch.testing.assert_close(pm.shared_expert(x, w, "m."), 0.5 * s)
    w["m.shared_expert_gate.weight"] = randn(1, h, seed=42)
    torch.testing.assert_close(pm.shared_expert(x, w, "m."),
                               torch.sigmoid(x @ w["m.shared_expert_gate.weight"].T) * s)


# ---- layer kinds and the whole model ---------------------------------------------
def test_layer_kinds_of_the_two_tiny_configurations():
    assert [pm.layer_is_sparse(CONFIG_A, l) for l in range(2)] == [True, True]
    assert [pm.layer_is_sparse(CONFIG_B, l) for l in range(3)] == [False, True, False]
    assert [pm.layer_window(CONFIG_B, l) for l in range(3)] == [None, None, 24]
    assert pm.layer_window(CONFIG_A, 1) is None


@pytest.fixture(scope="module")
def model_b(model_dirs):
    import util
    return util.read_folder(model_dirs["B"]["float32"])


def test_model_is_causal(model_b):
    cfg, w = model_b
    toks = list(range(3, 40))
    full = pm.forward(w, cfg, toks)
    torch.testing.assert_close(pm.forward(w, cfg, toks[:20]), full[:20], atol=1e-5, rtol=1e-5)


def test_shifting_all_positions_changes_nothing(model_b):
    """Only distances between positions count (rotary + causal + window)."""
    cfg, w = model_b
    toks = list(range(50, 80))
    torch.testing.assert_close(pm.forward(w, cfg, toks, first_position=1000),
                               pm.forward(w, cfg, toks), atol=2e-3, rtol=2e-3)


def test_window_matters_and_tied_head_is_the_embedding(model_b):
    cfg, w = model_b
    toks = list(range(100, 140))
    full = pm.forward(w, cfg, toks)
    no_window = dict(cfg, use_sliding_window=False)
    other = pm.forward(w, no_window, toks)
    torch.testing.assert_close(other[:24], full[:24])      # first 24 rows see everything anyway
    assert (other[30:] - full[30:]).abs().max() > 1e-4
    assert "lm_head.weight" not in w


def test_plan_with_shared_cache_differs_from_default(model_b):
    cfg, w = model_b
    toks = list(range(7, 30))
    default = pm.forward(w, cfg, toks)
    shared = pm.forward(w, cfg, toks, plan=[(0, None), (1, 0), (2, None)])
    assert (default - shared).abs().max() > 1e-4
    twice = pm.forward(w, cfg, toks, plan=[(0, None), (1, None), (1, None), (2, None)])
    assert twice.shape == default.shape and (default - twice).abs().max() > 1e-4


def test_sampling_distribution_limits():
    l = randn(50, seed=50) * 2
    p = pm.sample_distribution(l, 0.0, 0, 1.0, 1.0, [])
    assert p.argmax() == l.argmax() and p.sum() == 1
    p1 = pm.sample_distribution(l, 1.0, 1, 1.0, 1.0, [])
    assert torch.equal(p, p1)                                  # top_k = 1 is greedy
    torch.testing.assert_close(pm.sample_distribution(l, 0.5, 0, 1.0, 1.0, []),
                               torch.softmax(l / 0.5, 0))
    p = pm.sample_distribution(l, 1.0, 10, 1.0, 1.0, [])
    assert (p > 0).sum() == 10
    p = pm.sample_distribution(l, 1.0, 0, 0.5, 1.0, [])
    kept = torch.softmax(l, 0)[p > 0]
    assert kept.sum() >= 0.5 and kept.sum() - kept.min() < 0.5  # shortest prefix reaching top_p
    rep = pm.sample_distribution(l, 1.0, 0, 1.0, 2.0, [int(l.argmax())])
    assert rep[l.argmax()] < torch.softmax(l, 0)[l.argmax()]
