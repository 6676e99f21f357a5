"""The engine's C interface (csrc/engine_api): through ctypes inside this process (the
library joins the running interpreter), and from a host program in C that a test compiles
and runs (the library starts an interpreter of its own). Same names and return codes as the
reference's C API (src/api/ninfer_c_api.h:32-82); what the functions return is compared with
the Python entry point and the plain model."""
import ctypes
import os
import subprocess
import sys

import numpy as np
import pytest

import plain_model
import util

pytestmark = pytest.mark.gpu


class Options(ctypes.Structure):
    _fields_ = [("max_context", ctypes.c_int), ("prefill_chunk", ctypes.c_int),
                ("num_sequences", ctypes.c_int), ("gpu_count", ctypes.c_int),
                ("gpus", ctypes.c_void_p), ("quant", ctypes.c_char_p), ("parallel", ctypes.c_char_p)]


@pytest.fixture(scope="module")
def lib():
    from ninfer_amd.kernels.build import engine_library
    path = engine_library()
    assert os.path.isfile(path), "the engine's C interface is not built"
    lib = ctypes.CDLL(path)
    lib.ninfer_last_error.restype = ctypes.c_char_p
    lib.ninfer_session_create.restype = ctypes.c_void_p
    lib.ninfer_sample.restype = ctypes.c_longlong
    lib.ninfer_request_add.restype = ctypes.c_longlong
    for name in ("ninfer_kv_bytes_per_token", "ninfer_kv_total_bytes", "ninfer_kv_seq_stride_elems",
                 "ninfer_kv_pages_total", "ninfer_kv_pages_free", "ninfer_kv_pages_reused"):
        getattr(lib, name).restype = ctypes.c_longlong
    return lib


def test_c_interface_in_process(lib, model_dirs):
    import ninfer_amd
    d = model_dirs["B"]["float32"]
    cfg, w = util.read_folder(d)
    vocab = cfg["vocab_size"]
    eng = ctypes.c_void_p()
    opt = Options(96, 8, 3, 1, None, b"f32", b"pp")
    assert lib.ninfer_load(d.encode(), ctypes.byref(opt), ctypes.byref(eng)) == 0, lib.ninfer_last_error()
    assert lib.ninfer_vocab_size(eng) == vocab and lib.ninfer_max_context(eng) == 96
    assert lib.ninfer_num_sequences(eng) == 3 and lib.ninfer_device_count(eng) == 1
    py = ninfer_amd.Ninfer(d, max_context=96, prefill_chunk=8, num_sequences=3, dtype="float32")
    assert lib.ninfer_kv_bytes_per_token(eng) == py.kv_bytes_per_token
    assert lib.ninfer_kv_total_bytes(eng) == py.kv_total_bytes
    assert lib.ninfer_kv_seq_stride_elems(eng) == 0

    prompt = util.safe_prompt(w, cfg, 19, 3)
    toks = (ctypes.c_longlong * len(prompt))(*prompt)
    logits = (ctypes.c_float * vocab)()
    s = ctypes.c_void_p(lib.ninfer_session_create(eng))
    assert s and lib.ninfer_session_length(s) == 0 and 0 <= lib.ninfer_session_slot(s) < 3
    assert lib.ninfer_prefill(s, toks, len(prompt), logits, vocab - 1) == -3
    assert lib.ninfer_session_length(s) == 0, "a refused call feeds nothing"
    assert lib.ninfer_prefill(s, toks, len(prompt), logits, vocab) == 0, lib.ninfer_last_error()
    with py.session() as ps:
        ref = ps.prefill(prompt)
        np.testing.assert_array_equal(np.ctypeslib.as_array(logits), ref)
        plain = plain_model.forward(w, cfg, prompt)[-1].numpy()
        np.testing.assert_allclose(ref, plain, atol=3e-5, rtol=1e-4)
        # greedy through ninfer_sample (temperature 0), token by token
        out = []
        for _ in range(6):
            t = lib.ninfer_sample(eng, logits, ctypes.c_float(0.0), 0, ctypes.c_float(1.0),
                                  ctypes.c_float(1.0), ctypes.c_ulonglong(0))
            assert t == int(np.argmax(np.ctypeslib.as_array(logits)))
            out.append(t)
            assert lib.ninfer_decode(s, ctypes.c_longlong(t), logits, vocab) == 0
        assert out == plain_model.greedy_generate(w, cfg, prompt, 6)
    assert lib.ninfer_session_length(s) == len(prompt) + 6
    # seeded sampling is the Python entry point's
    t1 = lib.ninfer_sample(eng, logits, ctypes.c_float(0.9), 20, ctypes.c_float(0.9),
                           ctypes.c_float(1.1), ctypes.c_ulonglong(77))
    assert t1 == py.sample(np.ctypeslib.as_array(logits), 0.9, 20, 0.9, 1.1, 77)
    # a mixed step: a portion of a second request's prompt beside the first one's next token
    t_next = int(np.argmax(np.ctypeslib.as_array(logits)))
    other = util.random_tokens(5, vocab, 8)
    s2 = ctypes.c_void_p(lib.ninfer_session_create(eng))
    sessions = (ctypes.c_void_p * 2)(s, s2)
    q_len = (ctypes.c_int * 2)(1, 5)
    flat = (ctypes.c_longlong * 6)(t_next, *other)
    rows = (ctypes.c_int * 3)(0, 2, 5)
    out3 = (ctypes.c_float * (3 * vocab))()
    assert lib.ninfer_step(eng, sessions, q_len, 2, flat, rows, 3, out3, 3 * vocab - 1) == -3
    assert lib.ninfer_step(eng, sessions, q_len, 2, flat, rows, 3, out3, 3 * vocab) == 0, lib.ninfer_last_error()
    got = np.ctypeslib.as_array(out3).reshape(3, vocab)
    ref_a = plain_model.forward(w, cfg, prompt + out + [t_next])[-1].numpy()
    ref_b = plain_model.forward(w, cfg, other).numpy()
    np.testing.assert_allclose(got[0], ref_a, atol=3e-5, rtol=1e-4)
    np.testing.assert_allclose(got[1:], ref_b[[1, 4]], atol=3e-5, rtol=1e-4)
    assert lib.ninfer_step(eng, sessions, q_len, 2, flat, None, 0, None, 0) == 0   # no logits wanted
    assert lib.ninfer_session_length(s2) == 10
    rows_bad = (ctypes.c_int * 2)(3, 1)
    assert lib.ninfer_step(eng, sessions, q_len, 2, flat, rows_bad, 2, out3, 3 * vocab) == -1
    lib.ninfer_session_free(s2)
    # what the engine holds under a checkpoint name
    name = "model.norm.weight"
    buf = (ctypes.c_float * 7)()
    assert lib.ninfer_tensor_read(eng, name.encode(), ctypes.c_longlong(3), ctypes.c_longlong(7), buf) == 0
    np.testing.assert_array_equal(np.ctypeslib.as_array(buf), w[name].float().numpy()[3:10])
    assert lib.ninfer_tensor_read(eng, b"no.such.tensor", ctypes.c_longlong(0), ctypes.c_longlong(1), buf) == -1
    total = lib.ninfer_kv_pages_total(eng)
    assert total == py.kv_pages()["total"] and 0 < lib.ninfer_kv_pages_free(eng) < total
    assert lib.ninfer_kv_pages_reused(eng) >= 0
    # errors: a message and a negative code, and the engine goes on
    bad = (ctypes.c_longlong * 2)(vocab + 5, 1)
    assert lib.ninfer_prefill(s, bad, 2, logits, vocab) == -1
    assert b"token" in lib.ninfer_last_error().lower()
    assert lib.ninfer_tokenize(eng, b"text", None, 0) == -1
    lib.ninfer_session_reset(s)
    assert lib.ninfer_session_length(s) == 0
    lib.ninfer_session_free(s)
    assert lib.ninfer_kv_pages_free(eng) == total
    # the scheduler through the C interface gives what the Python entry point's gives: seeded
    # sampling, a stop token, a request that can never fit
    prompts = [util.safe_prompt(w, cfg, n, 40 + n) for n in (9, 21, 14)]
    params = ninfer_amd.SamplingParams(0.8, 20, 0.9, 1.05, 123, 7)
    ids = []
    for p in prompts:
        arr = (ctypes.c_longlong * len(p))(*p)
        ids.append(lib.ninfer_request_add(eng, arr, len(p), 7, ctypes.c_float(0.8), 20, ctypes.c_float(0.9),
                                          ctypes.c_float(1.05), ctypes.c_ulonglong(123), None, 0))
    assert ids == [0, 1, 2]
    long_prompt = (ctypes.c_longlong * 95)(*([1] * 95))
    too_long = lib.ninfer_request_add(eng, long_prompt, 95, 7, ctypes.c_float(0.0), 0, ctypes.c_float(1.0),
                                      ctypes.c_float(1.0), ctypes.c_ulonglong(0), None, 0)
    while lib.ninfer_run_step(eng) > 0:
        pass
    want = py.generate(prompts, params, stop_ids=[])
    outbuf = (ctypes.c_longlong * 16)()
    for rid, ref_tokens in zip(ids, want):
        assert lib.ninfer_request_take(eng, ctypes.c_longlong(rid), outbuf, 3) == -3
        n = lib.ninfer_request_take(eng, ctypes.c_longlong(rid), outbuf, 16)
        assert list(outbuf[:n]) == ref_tokens
    assert lib.ninfer_request_take(eng, ctypes.c_longlong(too_long), outbuf, 16) == -1
    assert b"max_context" in lib.ninfer_last_error()
    assert lib.ninfer_request_take(eng, ctypes.c_longlong(99), outbuf, 16) == -1
    lib.ninfer_engine_free(eng)
    eng2 = ctypes.c_void_p()
    for quant, parallel, gpus in ((b"q4", None, 1), (None, b"tp", 1), (None, None, 2)):
        opt = Options(96, 8, 1, gpus, None, quant, parallel)
        assert lib.ninfer_load(d.encode(), ctypes.byref(opt), ctypes.byref(eng2)) == -1
        assert lib.ninfer_last_error()
    py.close()


def test_c_interface_from_a_c_program(model_dirs, tmp_path):
    """A host program in C, compiled here against the header and the library: the library
    starts an interpreter of its own inside it."""
    from ninfer_amd.kernels.build import CSRC, engine_library
    d = model_dirs["A"]["float32"]
    cfg, w = util.read_folder(d)
    lib_dir = os.path.dirname(engine_library())
    exe = str(tmp_path / "c_api_host")
    src = os.path.join(os.path.dirname(os.path.abspath(__file__)), "c_api_host.c")
    subprocess.run(["gcc", "-O1", "-std=c11", "-I", os.path.join(CSRC, "engine_api"), src, "-o", exe,
                    f"-L{lib_dir}", f"-Wl,-rpath,{lib_dir}", "-lninfer_engine"], check=True)
    prompt = util.safe_prompt(w, cfg, 13, 9)
    env = dict(os.environ, PYTHONPATH="")
    p = subprocess.run([exe, d, "5"] + [str(t) for t in prompt], capture_output=True, text=True,
                       timeout=280, env=env)
    assert p.returncode == 0, p.stdout + p.stderr
    lines = dict(l.split(":", 1) for l in p.stdout.strip().splitlines())
    want = plain_model.greedy_generate(w, cfg, prompt, 5)
    assert [int(t) for t in lines["a"].split()] == want
    assert [int(t) for t in lines["batch"].split()] == want
    assert [int(t) for t in lines["scheduled"].split()] == want
    assert int(lines["pages"]) > 0
