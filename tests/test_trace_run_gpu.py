"""bin/trace_run as a user calls it: a subprocess fed JSON lines, logits read
back from <step>.f32 files. The same requests are replayed whole, with the last
32 tokens one by one, in portions of changing size, and mixed with other
requests so that pages are used again; in 32-bit and in bfloat16; all are
compared with the plain implementation."""
import os
import subprocess
import sys

import pytest
import torch

import plain_model
import util
from conftest import ROOT, TINY

pytestmark = pytest.mark.gpu

LENS = {"A": [17, 45, 60, 38], "B": [15, 52, 70, 45, 33], "C": [20, 66, 90, 41]}


def replay(model_dir, dtype, steps, out_dir, max_tokens, vocab):
    proc = subprocess.run(
        [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model_dir, "--dtype",
         dtype, "--out", out_dir, "--max-tokens", str(max_tokens)],
        input=util.write_trace(steps), capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    done = [l for l in proc.stdout.splitlines() if l.startswith("done ")]
    assert done == [f"done {i}" for i in range(len(steps))]
    return util.read_trace_output(out_dir, steps, vocab)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_trace_replay_all_ways(model_dirs, tmp_path, name, dtype):
    d = model_dirs[name][dtype]
    cfg, w = util.read_folder(d)
    _, w16 = util.read_folder(model_dirs[name]["bfloat16"])
    reqs = {f"q{i}": util.safe_prompt(w16, cfg, n, 300 + i) for i, n in enumerate(LENS[name])}
    ref = {k: plain_model.forward(w, cfg, v) for k, v in reqs.items()}
    bound = dict(atol=2e-5, rtol=1e-4) if dtype == "float32" else dict(atol=6e-2, rtol=5e-2)
    vocab = cfg["vocab_size"]
    # every request alone: whole, tail of 32 one by one, changing portions; one process for all
    steps = []
    for k, v in reqs.items():
        for tag, sched in (("w", util.schedule_whole(k, v)), ("t", util.schedule_tail(k, v, 32)),
                           ("p", util.schedule_portions(k, v, len(v)))):
            steps += [([(r + tag, t, want) for r, t, want in e], [r + tag for r in end])
                      for e, end in sched]
    got = replay(d, dtype, steps, str(tmp_path / "alone"), 128, vocab)
    for k in reqs:
        for tag in "wtp":
            torch.testing.assert_close(got[k + tag], ref[k], **bound,
                                       msg=lambda m: f"{name} {dtype} {k}{tag}: {m}")
    # mixed: up to four live; 256 tokens of pool for ~215 tokens in flight: pages come back
    steps = util.schedule_mixed(reqs, seed=11, max_live=4)
    got = replay(d, dtype, steps, str(tmp_path / "mixed"), 256, vocab)
    for k in reqs:
        torch.testing.assert_close(got[k], ref[k], **bound,
                                   msg=lambda m: f"{name} {dtype} {k} mixed: {m}")
    import json
    with open(str(tmp_path / "mixed" / "stats.json")) as f:
        stats = json.load(f)
    assert stats["steps"] == len(steps) and len(stats["groups"]) == (1 if name == "A" else 2)
    for g in stats["groups"]:
        assert g["reused"] > 0 and g["in_use"] == 0 and g["allocated"] == g["freed"]
        assert 0 < g["peak_in_use"] <= g["pages"] == 16
        assert (g["window_freed"] > 0) == (g["window"] is not None)
