"""Paged attention at the context lengths and batch shapes that serving and the
benchmark run (2,048 to 32,768 keys, 8 and 64 decoded rows, 16 kv heads and 28
query heads on 4 kv heads), against the plain twin (tests/plain_ops.py).

With few rows and short contexts the split-context kernels always cut the
context into chunks of 128 keys; the larger chunks (256 for the scalar kernel from 24 blocks a CU on,
256, 512 and 1,024 for the matrix-core kernel of grouped heads) and a merge over
a hundred and more chunks are reached only by the shapes here. Each case first
asks the library which kernel and chunk size it would run and asserts that it is
the variant the case is meant for.

Random keys alone would hide a dropped chunk (the output of attention over
thousands of random keys is close to the mean of the values whatever is left
out), so the queries are scaled until a handful of keys, at random places,
carry most of each row's weight; and one key at a chosen place (a chunk's first
or last key, the context's first and last) is made to dominate a row, whose
output must then be that key's value.

All requests of a case share one long stream of keys (their block tables name
the same pages, each as far as its own length): 32,768 keys are stored once.
"""
import math
from types import SimpleNamespace

import pytest
import torch

from plain_ops import PlainOps

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from ninfer_amd.kernels import load_ops
    return load_ops()


def tol(dtype):
    return (2e-5, 1e-4) if dtype == torch.float32 else (2e-2, 2e-2)


def shared_stream_case(seqs, n_q, n_kv, d, ps, dtype, window=0, q_scale=4.0, seed=7):
    """seqs: (first position, rows) per request. One stream of keys and values as long as
    the longest request; every request's block table names the stream's pages up to its own
    length, without those a window has wholly passed."""
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    longest = max(p + q for p, q in seqs)
    n_pages = -(-longest // ps)
    perm = torch.randperm(n_pages + 5, generator=torch.Generator().manual_seed(seed))
    bt = torch.full((len(seqs), n_pages), -1, dtype=torch.int32)
    for i, (p, q) in enumerate(seqs):
        held = -(-(p + q) // ps)
        bt[i, :held] = perm[:held].to(torch.int32)
        if window:
            dead = (p - window + 1) // ps   # pages that every row of the request has passed
            if dead > 0:
                bt[i, :dead] = -1
    rnd = lambda *shape: torch.randn(*shape, generator=g, device="cuda")
    k_pool = rnd(n_pages + 5, n_kv, ps, d).to(dtype)
    v_pool = rnd(n_pages + 5, n_kv, ps, d).to(dtype)
    positions, row_seq, row_start = [], [], []
    for i, (p, q) in enumerate(seqs):
        row_start.append(len(positions))
        positions += list(range(p, p + q))
        row_seq += [i] * q
    row_start.append(len(positions))
    dev = lambda x: torch.tensor(x, dtype=torch.int32, device="cuda")
    ctx = SimpleNamespace(S=len(seqs), T=len(positions), positions=dev(positions),
                          row_seq=dev(row_seq), seq_row_start=dev(row_start),
                          seq_qlen=dev([q for _, q in seqs]), seq_pos0=dev([p for p, _ in seqs]),
                          max_qlen=max(q for _, q in seqs), max_kv_len=longest)
    qkv = (rnd(ctx.T, (n_q + 2 * n_kv) * d) * q_scale).to(dtype)
    return ctx, qkv, k_pool, v_pool, bt.cuda(), perm


def place_dominant_key(qkv, k_pool, perm, row, key, n_q, n_kv, d, ps, dtype):
    """Key `key` of the stream becomes a vector of +-1 and every query head of `row` 16 times
    that vector: its score is 16 sqrt(d), far above every other key's."""
    page, slot = int(perm[key // ps]), key % ps
    k_pool[page, :, slot, :] = torch.sign(k_pool[page, :, slot, :].float() + 1e-3).to(dtype)
    group = n_q // n_kv
    for h in range(n_q):
        qkv[row, h * d:(h + 1) * d] = (16 * k_pool[page, h // group, slot, :].float()).to(dtype)
    return page, slot


def run_both(ops, case, n_q, n_kv, d, ps, window, dtype):
    ctx, qkv, k_pool, v_pool, bt, _ = case
    o1 = torch.empty(ctx.T, n_q * d, device="cuda", dtype=dtype)
    o2 = torch.empty_like(o1)
    scale = 1 / math.sqrt(d)
    ops.paged_attention(qkv, k_pool, v_pool, bt, ctx, n_q, n_kv, d, ps, window, scale, o1)
    PlainOps().paged_attention(qkv, k_pool, v_pool, bt, ctx, n_q, n_kv, d, ps, window, scale, o2)
    return o1, o2


# Decoded rows. name: (heads, kv heads, head size, page, window, last positions of the rows,
# the kernel, chunk size and least number of chunks the case is for)
DECODE_CASES = {
    # 8 rows x 16 kv heads over 8,192 keys: the benchmark's default step
    "scalar128-b8-8k": (16, 16, 128, 16, 0,
                        [8191, 8192, 8447, 8448, 5000, 255, 256, 0], "scalar", 128, 67),
    # the same with 32 rows: blocks enough for the larger chunks
    "scalar256-b32-8k": (16, 16, 128, 16, 0,
                         [8191, 8192, 8447, 8448, 5000, 255, 256, 0] * 4, "scalar", 256, 34),
    # 64 rows over about 2,048 keys, contexts that end at, before and after chunk edges
    "scalar256-b64-2k": (16, 16, 128, 16, 0,
                         [2047, 2048, 2049, 2303, 2304, 1023, 1024, 1100, 511, 512, 767, 768, 3,
                          16, 17, 1999] * 4, "scalar", 256, 10),
    # 32,768 keys: the merge kernel adds up 128 chunks
    "scalar256-b8-32k": (16, 16, 128, 16, 0,
                         [32767, 32766, 32512, 32511, 20000, 16384, 300, 31], "scalar", 256, 128),
    # one row, two kv heads: the GPU is not filled, chunks of 128, 256 of them to merge
    "scalar128-b1-32k": (4, 2, 64, 16, 0, [32767], "scalar", 128, 256),
    # a window whose first key lies inside a chunk and inside a page
    "scalar128-b8-8k-window": (16, 16, 128, 16, 4000,
                               [8191, 8192, 8447, 8448, 5000, 255, 4000, 3999], "scalar", 128, 67),
    "scalar256-b32-8k-window": (16, 16, 128, 16, 4000,
                                [8191, 8192, 8447, 8448, 5000, 255, 4000, 3999] * 4, "scalar", 256, 34),
    "scalar256-b64-d64-window": (8, 8, 64, 32, 1500,
                                 [4095, 4096, 2047, 1499, 1500, 1501, 3000, 2999] * 8,
                                 "scalar", 256, 17),
    # 28 query heads on 4 kv heads (the larger model of the family): the matrix-core kernel
    "heads1024-b8-32k": (28, 4, 128, 16, 0,
                         [32767, 32766, 31744, 31743, 20000, 1024, 1023, 5], "heads", 1024, 32),
    "heads512-b8-8k": (28, 4, 128, 16, 0,
                       [8191, 8190, 7680, 7679, 512, 511, 3000, 0], "heads", 512, 16),
    "heads256-b8-4k": (28, 4, 128, 16, 0,
                       [4095, 4094, 3840, 3839, 256, 255, 1000, 77], "heads", 256, 16),
    "heads1024-b64-2k": (28, 4, 128, 16, 0,
                         [2099, 2047, 2048, 1023, 1024, 1025, 100, 2000] * 8, "heads", 1024, 3),
    "heads1024-b64-8k-window": (28, 4, 128, 16, 3000,
                                [8191, 8192, 8200, 6143, 6144, 2999, 3000, 3001] * 8,
                                "heads", 1024, 9),
    "heads512-b8-8k-window": (28, 4, 128, 16, 700,
                              [8191, 8190, 7680, 7679, 512, 699, 700, 701], "heads", 512, 16),
    # heads of 64 in groups of three
    "heads256-d64-b8-4k": (12, 4, 64, 64, 0,
                           [4095, 4000, 2048, 2047, 300, 256, 255, 3], "heads", 256, 16),
    "heads512-d64-b16-4k": (12, 4, 64, 32, 0,
                            [4095, 4000, 2048, 2047, 300, 512, 511, 3] * 2, "heads", 512, 8),
    # one row of 8 heads on one kv head: chunks of 128, 256 of them
    "heads128-b1-32k": (8, 1, 128, 16, 0, [32767], "heads", 128, 256),
}


@pytest.mark.parametrize("name", sorted(DECODE_CASES))
def test_decode_rows_at_long_contexts(ops, name):
    n_q, n_kv, d, ps, window, last, kernel, chunk, min_chunks = DECODE_CASES[name]
    dtype = torch.bfloat16
    seqs = [(p, 1) for p in last]
    case = shared_stream_case(seqs, n_q, n_kv, d, ps, dtype, window)
    ctx, qkv, k_pool, v_pool, bt, perm = case
    out = torch.empty(ctx.T, n_q * d, device="cuda", dtype=dtype)
    plan = ops.paged_attention(qkv, k_pool, v_pool, bt, ctx, n_q, n_kv, d, ps, window,
                               1 / math.sqrt(d), out, plan_only=True)
    assert plan["kernel"] == kernel and plan["chunk"] == chunk and plan["chunks"] >= min_chunks, plan
    o1, o2 = run_both(ops, case, n_q, n_kv, d, ps, window, dtype)
    atol, rtol = tol(dtype)
    torch.testing.assert_close(o1.float().cpu(), o2.float().cpu(), atol=atol, rtol=rtol)
    # the rows are not near the mean of the values: what they see matters
    assert float(o2.float().abs().mean()) > 0.1


@pytest.mark.parametrize("name", ["scalar128-b8-8k", "scalar256-b32-8k", "scalar256-b8-32k",
                                  "heads1024-b8-32k", "heads512-b8-8k", "heads256-b8-4k",
                                  "scalar128-b8-8k-window", "scalar256-b32-8k-window",
                                  "heads512-b8-8k-window"])
def test_decode_rows_find_one_key_at_chunk_edges(ops, name):
    """Row 0 (the longest context of the case) is made to look for one key: the context's
    first and last, and the keys on both sides of a chunk's edge near the start, the
    middle and the end. Inside the window its value must come out; the key that the window
    has just passed must not be seen."""
    n_q, n_kv, d, ps, window, last, kernel, chunk, _ = DECODE_CASES[name]
    dtype = torch.bfloat16
    pos = last[0]
    lo = max(0, pos - window + 1) if window else 0
    mid = (lo + pos) // 2 // chunk * chunk
    keys = sorted({lo, lo + 1, pos, pos - 1, mid - 1, mid, (pos // chunk) * chunk,
                   (pos // chunk) * chunk - 1, -(-lo // chunk) * chunk, -(-lo // chunk) * chunk - 1})
    keys = [k for k in keys if lo <= k <= pos]
    group = n_q // n_kv
    for key in keys + ([lo - 1] if lo > 0 else []):
        case = shared_stream_case([(p, 1) for p in last], n_q, n_kv, d, ps, dtype, window)
        ctx, qkv, k_pool, v_pool, bt, perm = case
        page, slot = place_dominant_key(qkv, k_pool, perm, 0, key, n_q, n_kv, d, ps, dtype)
        out = torch.empty(ctx.T, n_q * d, device="cuda", dtype=dtype)
        ops.paged_attention(qkv, k_pool, v_pool, bt, ctx, n_q, n_kv, d, ps, window,
                            1 / math.sqrt(d), out)
        for h in range(n_q):
            got = out[0, h * d:(h + 1) * d].float()
            value = v_pool[page, h // group, slot, :].float()
            if key >= lo:
                torch.testing.assert_close(got, value, atol=2e-2, rtol=2e-2,
                                           msg=f"{name}: key {key} of {lo}..{pos} not found")
            else:
                assert (got - value).abs().max() > 0.2, f"{name}: key {key} outside the window was seen"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "f32"])
@pytest.mark.parametrize("window", [0, 5000])
def test_prompt_portion_behind_a_long_context(ops, dtype, window):
    """2,048 rows of one request behind 30,720 cached keys (the last portion of a 32,768-token
    prompt), beside a short request and a decoded row of a third: block tables of 2,048 pages,
    480 key tiles before the portion's own."""
    n_q, n_kv, d, ps = 4, 2, 128, 16
    seqs = [(30720, 2048), (0, 70), (12345, 1)]
    case = shared_stream_case(seqs, n_q, n_kv, d, ps, dtype, window, q_scale=4.0)
    o1, o2 = run_both(ops, case, n_q, n_kv, d, ps, window, dtype)
    atol, rtol = tol(dtype)
    torch.testing.assert_close(o1.float().cpu(), o2.float().cpu(), atol=atol, rtol=rtol)
    assert float(o2.float().abs().mean()) > 0.1
    # the same rows with the single-token request announced first (as the step function
    # orders them): it runs on the split-context kernel, the portions on the prompt kernel
    if dtype == torch.bfloat16:
        seqs2 = [(12345, 1), (30720, 2048), (0, 70)]
        case2 = shared_stream_case(seqs2, n_q, n_kv, d, ps, dtype, window, q_scale=4.0)
        case2[0].single_rows = 1
        a, b = run_both(ops, case2, n_q, n_kv, d, ps, window, dtype)
        torch.testing.assert_close(a.float().cpu(), b.float().cpu(), atol=atol, rtol=rtol)


def test_prompt_rows_find_one_key_far_back(ops):
    """Rows of a portion behind 30,720 keys look for single keys: the stream's first, one
    on each side of a tile of 64 far back, the row's own position."""
    n_q, n_kv, d, ps, dtype = 4, 2, 128, 16, torch.bfloat16
    seqs = [(30720, 256)]
    for row, key in ((0, 0), (255, 63), (100, 64), (17, 20479), (200, 20480), (31, 30751),
                     (128, 30720 + 128), (129, 30720 + 127)):
        case = shared_stream_case(seqs, n_q, n_kv, d, ps, dtype, 0)
        ctx, qkv, k_pool, v_pool, bt, perm = case
        page, slot = place_dominant_key(qkv, k_pool, perm, row, key, n_q, n_kv, d, ps, dtype)
        out = torch.empty(ctx.T, n_q * d, device="cuda", dtype=dtype)
        ops.paged_attention(qkv, k_pool, v_pool, bt, ctx, n_q, n_kv, d, ps, 0, 1 / math.sqrt(d), out)
        for h in range(n_q):
            torch.testing.assert_close(out[row, h * d:(h + 1) * d].float(),
                                       v_pool[page, h // 2, slot, :].float(), atol=2e-2, rtol=2e-2,
                                       msg=f"row {row}: key {key} not found")
