"""Each part alone on the GPU (norm, position encoding + attention mixer, dense
feed-forward, sparse feed-forward, block), built from its parameters and bound
to random weights, against the plain function for that part; at sizes other
than the tiny models'."""
import math

import pytest
import torch

import plain_model as pm
import util

pytestmark = pytest.mark.gpu

BOUND = {torch.float32: dict(atol=3e-5, rtol=1e-4), torch.bfloat16: dict(atol=5e-2, rtol=5e-2)}


@pytest.fixture(scope="module")
def ops():
    from ninfer_amd.kernels import load_ops
    return load_ops()


def bind(part, weights, dtype):
    from ninfer_amd.parts import WeightBinder
    part.bind_all(WeightBinder(util.DictSource(weights), torch.device("cuda"), dtype))


def rounded(weights, dtype):
    """The values the part actually holds (matrices rounded to the compute dtype)."""
    return {k: (v.to(dtype).float() if v.dim() > 1 else v) for k, v in weights.items()}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rmsnorm_part(ops, dtype):
    from ninfer_amd.parts import RMSNorm
    norm = RMSNorm("n.", 200, 1e-5)
    w = util.random_part_weights(norm, 1)
    bind(norm, w, dtype)
    ctx = util.make_context(ops, dtype, [(0, 7)])
    x = torch.randn(7, 200, device="cuda") * 2
    pending = torch.randn(7, 200, device="cuda").to(dtype)
    ref = pm.rms_norm((x + pending.float()).cpu(), w["n.weight"], 1e-5)
    out = norm.forward(ctx, x, pending)
    torch.testing.assert_close(out.float().cpu(), ref, **BOUND[dtype])
    torch.testing.assert_close(x.cpu(), (x.cpu()), atol=0, rtol=0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv,d,window", [(6, 2, 48, None), (4, 4, 64, 20), (8, 1, 128, None)])
def test_attention_part(ops, dtype, heads, kv, d, window):
    """Rotary + attention over pages, fed in two portions, against the plain
    whole-sequence attention."""
    from ninfer_amd.parts import Attention, CacheView, CallInfo, Rotary
    hidden, t, ps = 72, 50, 8
    att = Attention("a.", hidden, heads, kv, d, Rotary(d, 1e5), qkv_bias=True, window=window)
    w = util.random_part_weights(att, 2)
    bind(att, w, dtype)
    wr = rounded(w, dtype)
    x = (torch.randn(t, hidden) * 0.5).to(dtype)
    pos = torch.arange(t)
    q, k, v = pm.attention_qkv(x.float(), wr, "a.", heads, kv, d, 1e5, pos)
    ref = pm.attention_core(q, k, v, pos, pos, window).reshape(t, heads * d) @ wr["a.o_proj.weight"].T
    n_pages = -(-t // ps)
    pools = [torch.zeros(n_pages + 2, kv, ps, d, device="cuda", dtype=dtype) for _ in range(2)]
    table = torch.arange(n_pages + 1, 0, -1, dtype=torch.int32, device="cuda")[None, :n_pages]
    outs = []
    for first, rows in ((0, 33), (33, 17)):
        ctx = util.make_context(ops, dtype, [(first, rows)])
        call = CallInfo(cache=CacheView({"k": pools[0], "v": pools[1]}, table.contiguous(), ps, window))
        outs.append(att.forward(ctx, x[first:first + rows].cuda(), None, call))
    got = torch.cat(outs).float().cpu()
    torch.testing.assert_close(got, ref, **BOUND[dtype])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_feed_forward_parts(ops, dtype):
    from ninfer_amd.parts import SparseMoE, SwiGLU
    hidden, t = 96, 21
    ctx = util.make_context(ops, dtype, [(0, t)])
    x = (torch.randn(t, hidden) * 0.7).to(dtype)
    dense = SwiGLU("m.", hidden, 160)
    w = util.random_part_weights(dense, 3)
    bind(dense, w, dtype)
    wr = rounded(w, dtype)
    ref = pm.swiglu_mlp(x.float(), wr["m.gate_proj.weight"], wr["m.up_proj.weight"],
                        wr["m.down_proj.weight"])
    torch.testing.assert_close(dense.forward(ctx, x.cuda(), None).float().cpu(), ref, **BOUND[dtype])
    for renorm in (False, True):
        moe = SparseMoE("m.", hidden, experts=6, top_k=2, inner=64, renorm=renorm, shared_inner=128)
        w = util.random_part_weights(moe, 4)
        bind(moe, w, dtype)
        wr = rounded(w, dtype)
        ids, wts = pm.router(x.float(), wr["m.gate.weight"], 2, renorm)
        if dtype == torch.bfloat16:   # keep rows whose routing is clear of rounding noise
            logits = x.float() @ wr["m.gate.weight"].T
            top = logits.sort(-1, descending=True).values
            clear = (top[:, 1] - top[:, 2]) > 0.05 * logits.abs().max(-1).values
        else:
            clear = torch.ones(t, dtype=torch.bool)
        ref = pm.routed_experts(x.float(), ids, wts, wr, "m.") + pm.shared_expert(x.float(), wr, "m.")
        from ninfer_amd.parts import PendingRows, RMSNorm
        residual = torch.zeros(t, hidden, device="cuda")
        pending = moe.forward(ctx, x.cuda(), residual)
        assert isinstance(pending, PendingRows)       # left for the next norm's kernel to add
        norm = RMSNorm("n.", hidden, 1e-6)
        bind(norm, {"n.weight": torch.ones(hidden)}, dtype)
        normed = norm.forward(ctx, residual, pending)   # adds on the fly, keeps the sum
        torch.testing.assert_close(residual.cpu()[clear], ref[clear], **BOUND[dtype])
        torch.testing.assert_close(normed.float().cpu()[clear],
                                   pm.rms_norm(ref, torch.ones(hidden), 1e-6)[clear],
                                   **BOUND[dtype])
        residual2 = torch.zeros(t, hidden, device="cuda")
        pending.add_to(ctx, residual2)                  # the same sum by the stand-alone kernel
        torch.testing.assert_close(residual2, residual, atol=1e-6, rtol=1e-6)
        assert clear.sum() > t // 2


def test_block_arrangement(ops):
    """x + mixer(norm1(x)), then + ff(norm2(.)): norms before, sums after."""
    from ninfer_amd.parts import (Attention, CacheView, CallInfo, PreNormBlock, RMSNorm, Rotary,
                                  SwiGLU)
    hidden, heads, d, t, ps = 64, 4, 16, 19, 4
    block = PreNormBlock(RMSNorm("b.n1.", hidden, 1e-6),
                         Attention("b.att.", hidden, heads, 2, d, Rotary(d, 1e4)),
                         RMSNorm("b.n2.", hidden, 1e-6), SwiGLU("b.ff.", hidden, 96))
    w = util.random_part_weights(block, 6)
    bind(block, w, torch.float32)
    x = torch.randn(t, hidden)
    pos = torch.arange(t)
    a = pm.rms_norm(x, w["b.n1.weight"], 1e-6)
    q, k, v = pm.attention_qkv(a, w, "b.att.", heads, 2, d, 1e4, pos)
    h1 = x + pm.attention_core(q, k, v, pos, pos, None).reshape(t, heads * d) @ w["b.att.o_proj.weight"].T
    m = pm.rms_norm(h1, w["b.n2.weight"], 1e-6)
    ref = h1 + pm.swiglu_mlp(m, w["b.ff.gate_proj.weight"], w["b.ff.up_proj.weight"],
                             w["b.ff.down_proj.weight"])
    ctx = util.make_context(ops, torch.float32, [(0, t)])
    pools = [torch.zeros(6, 2, ps, d, device="cuda") for _ in range(2)]
    table = torch.arange(5, dtype=torch.int32, device="cuda")[None]
    residual = x.cuda().clone()
    pending = block.forward(ctx, residual, None, CallInfo(cache=CacheView({"k": pools[0], "v": pools[1]},
                                                                          table, ps, None)))
    torch.testing.assert_close((residual + pending).cpu(), ref, atol=3e-5, rtol=1e-4)
    torch.testing.assert_close(residual.cpu(), h1, atol=3e-5, rtol=1e-4)
