"""The entry point that allocates nothing (decode attention with its workspace in a fixed
device array of the library), called through ctypes as a caller without torch would, against
the existing entry point on the same arguments: two calls in a row, the second with a smaller
input (fewer rows, shorter contexts: it finds the first call's partial results in the array and
must not read them), then a larger one again; both split-context kernels; and a shape whose
workspace exceeds the array, which is refused."""
import ctypes
import math

import pytest
import torch

pytestmark = pytest.mark.gpu


def _case(last_positions, n_q, n_kv, d, ps, seed):
    """Single-token rows at the given positions, each request with pages of its own."""
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    s = len(last_positions)
    pages_of = [p // ps + 1 for p in last_positions]
    n_pages = sum(pages_of) + 2
    perm = torch.randperm(n_pages, generator=torch.Generator().manual_seed(seed)).tolist()
    bt = torch.full((s, max(pages_of)), -1, dtype=torch.int32)
    for i, n in enumerate(pages_of):
        for lp in range(n):
            bt[i, lp] = perm.pop()
    rnd = lambda *shape: torch.randn(*shape, generator=g, device="cuda").to(torch.bfloat16)
    dev = lambda x: torch.tensor(x, dtype=torch.int32, device="cuda")
    return dict(qkv=rnd(s, (n_q + 2 * n_kv) * d) * 3, k=rnd(n_pages, n_kv, ps, d),
                v=rnd(n_pages, n_kv, ps, d), bt=bt.cuda(), positions=dev(last_positions),
                row_seq=dev(list(range(s))), row_start=dev(list(range(s + 1))),
                qlen=dev([1] * s), pos0=dev(last_positions), max_kv_len=max(last_positions) + 1)


def _args(AttnArgs, c, out, n_q, n_kv, d, ps, window, workspace=None):
    s = c["qkv"].shape[0]
    return AttnArgs(
        c["qkv"].data_ptr(), c["k"].data_ptr(), c["v"].data_ptr(), out.data_ptr(),
        c["bt"].data_ptr(), c["positions"].data_ptr(), c["row_seq"].data_ptr(),
        c["row_start"].data_ptr(), c["qlen"].data_ptr(), c["pos0"].data_ptr(),
        workspace.data_ptr() if workspace is not None else None,
        workspace.numel() if workspace is not None else 0,
        c["qkv"].shape[1], c["bt"].shape[1], s, s, n_q, n_kv, d, ps, window, 1 / math.sqrt(d), 1, 1,
        c["max_kv_len"], 0)


@pytest.mark.parametrize("n_q,n_kv,d,ps,window,kernel", [(16, 16, 128, 16, 0, 1), (28, 4, 128, 16, 0, 2),
                                                         (6, 2, 64, 32, 300, 2)],
                         ids=["scalar", "heads", "heads-d64-window"])
def test_decode_attention_without_allocation(n_q, n_kv, d, ps, window, kernel):
    from ninfer_amd.kernels.build import ensure_built
    from ninfer_amd.kernels.ops import _AttnArgs
    lib = ctypes.CDLL(ensure_built())
    lib.ninfer_last_error.restype = ctypes.c_char_p
    lib.ninfer_attention_workspace_floats.restype = ctypes.c_longlong
    lib.ninfer_decode_attention_static_max_floats.restype = ctypes.c_longlong
    assert lib.ninfer_decode_attention_static_init() == 0, lib.ninfer_last_error().decode()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    # a warm call: whatever the library loads or maps at its first launch on the device (code
    # objects, the array's backing) has happened before device memory is watched below
    c = _case([70, 3], n_q, n_kv, d, ps, seed=2)
    warm = torch.zeros(2, n_q * d, dtype=torch.bfloat16, device="cuda")
    assert lib.ninfer_decode_attention_static(
        ctypes.byref(_args(_AttnArgs, c, warm, n_q, n_kv, d, ps, window)), stream) == 0
    torch.cuda.synchronize()
    calls = [[4000, 4095, 4096, 1023, 77, 2500, 0, 3999],   # 8 rows, contexts to 4,097 keys
             [300, 129, 5],                                  # smaller: 3 rows, 301 keys
             [900, 2047, 2048, 15, 16]]
    for i, last in enumerate(calls):
        c = _case(last, n_q, n_kv, d, ps, seed=11 + i)
        s = len(last)
        need = lib.ninfer_attention_workspace_floats(s, n_q, d, c["max_kv_len"])
        ws = torch.empty(need, dtype=torch.float32, device="cuda")
        want = torch.zeros(s, n_q * d, dtype=torch.bfloat16, device="cuda")
        got = torch.zeros_like(want)
        a = _args(_AttnArgs, c, want, n_q, n_kv, d, ps, window, ws)
        assert lib.ninfer_paged_attention(ctypes.byref(a), 0, stream) == 0, lib.ninfer_last_error().decode()
        b = _args(_AttnArgs, c, got, n_q, n_kv, d, ps, window)
        # the variant this case means to reach (1: scalar FMAs, 2: grouped heads on the matrix cores)
        which, chunk, chunks = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
        assert lib.ninfer_attention_decode_plan(ctypes.byref(a), ctypes.byref(which),
                                                ctypes.byref(chunk), ctypes.byref(chunks)) == 0
        assert which.value == kernel
        torch.cuda.synchronize()
        # free bytes of the device, not torch's own count: an allocation by the library
        # itself (hipMalloc, a lazily loaded code object) would show here
        before, held = torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated()
        rc = lib.ninfer_decode_attention_static(ctypes.byref(b), stream)
        assert rc == 0, lib.ninfer_last_error().decode()
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == before and torch.cuda.memory_allocated() == held
        assert want.float().abs().sum() > 0
        assert torch.equal(got, want), f"call {i}: the outputs differ"
    # a shape whose partial results do not fit the array is refused, and nothing runs
    limit = lib.ninfer_decode_attention_static_max_floats()
    c = _case([40000] * 2 + [5] * 62, n_q, n_kv, d, ps, seed=3)
    assert lib.ninfer_attention_workspace_floats(64, n_q, d, c["max_kv_len"]) > limit
    out = torch.full((64, n_q * d), 7.0, dtype=torch.bfloat16, device="cuda")
    rc = lib.ninfer_decode_attention_static(
        ctypes.byref(_args(_AttnArgs, c, out, n_q, n_kv, d, ps, window)), stream)
    assert rc != 0 and b"workspace" in lib.ninfer_last_error()
    torch.cuda.synchronize()
    assert (out == 7.0).all()
    # a position at or beyond max_kv_len (a caller's mistake) is read as the last one inside
    # the bound: the call stays inside the array and gives what the bound's context gives
    c = _case([600, 40], n_q, n_kv, d, ps, seed=5)
    want = torch.zeros(2, n_q * d, dtype=torch.bfloat16, device="cuda")
    got = torch.zeros_like(want)
    c["max_kv_len"] = 300
    c["positions"] = torch.tensor([299, 40], dtype=torch.int32, device="cuda")
    assert lib.ninfer_decode_attention_static(
        ctypes.byref(_args(_AttnArgs, c, want, n_q, n_kv, d, ps, window)), stream) == 0
    c["positions"] = torch.tensor([600, 40], dtype=torch.int32, device="cuda")
    assert lib.ninfer_decode_attention_static(
        ctypes.byref(_args(_AttnArgs, c, got, n_q, n_kv, d, ps, window)), stream) == 0
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    # prompt portions are not its business
    c = _case([10, 20], n_q, n_kv, d, ps, seed=4)
    bad = _args(_AttnArgs, c, torch.zeros(2, n_q * d, dtype=torch.bfloat16, device="cuda"),
                n_q, n_kv, d, ps, window)
    bad.max_qlen = 2
    assert lib.ninfer_decode_attention_static(ctypes.byref(bad), stream) != 0
