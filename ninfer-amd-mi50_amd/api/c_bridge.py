"""What the engine's C interface calls (csrc/engine_api/ninfer_c_api.cpp): one function per
C function, taking plain numbers. Pointers arrive as integers; tokens are read from and
logits written to the caller's memory through ctypes. Exceptions pass through: the C side
turns them into a negative return code and a message. Return codes follow the reference
(src/api/ninfer_c_api.cpp:171-246): 0, or -3 when the caller's buffer is too small.
"""
from __future__ import annotations

import ctypes
from typing import List

import numpy as np

from ..engine.scheduler import Request, Scheduler
from ..sampling.params import SamplingParams
from .ninfer import Ninfer, Session

_DTYPES = {None: "bfloat16", "": "bfloat16", "fp16": "bfloat16", "bf16": "bfloat16",
           "bfloat16": "bfloat16", "f32": "float32", "fp32": "float32", "float32": "float32"}


def load(model_dir: str, max_context: int, prefill_chunk: int, num_sequences: int,
         gpu_count: int, quant, parallel) -> Ninfer:
    """Defaults as the reference's ninfer_load (src/api/ninfer_c_api.cpp:61-64)."""
    if gpu_count not in (0, 1):
        raise ValueError(f"gpu_count {gpu_count}: this engine runs on one GPU")
    if parallel not in (None, "", "pp"):
        raise ValueError(f"parallel {parallel!r}: this engine runs on one GPU")
    if quant not in _DTYPES:
        raise ValueError(f"quant {quant!r}: one of 'fp16' / 'bf16' (both bfloat16) or 'f32'")
    return Ninfer(model_dir, max_context=max_context if max_context > 0 else 32768,
                  prefill_chunk=prefill_chunk if prefill_chunk > 0 else 512,
                  num_sequences=num_sequences if num_sequences > 0 else 1, dtype=_DTYPES[quant])


def close(engine: Ninfer) -> None:
    engine.close()


def engine_number(engine: Ninfer, what: str) -> int:
    if what == "pages_total":
        return int(engine.kv_pages()["total"])
    if what == "pages_free":
        return int(engine.kv_pages()["free"])
    if what == "pages_reused":
        return int(engine.kv_pages()["reused"])
    return int(getattr(engine, what))


def session(engine: Ninfer) -> Session:
    return engine.session()


def session_close(s: Session) -> None:
    s.close()


def session_reset(s: Session) -> None:
    s.reset()


def session_number(s: Session, what: str) -> int:
    return int(getattr(s, what))


def _tokens(address: int, count: int) -> List[int]:
    return list((ctypes.c_longlong * count).from_address(address))


def _write(logits: np.ndarray, address: int, capacity: int) -> int:
    flat = np.ascontiguousarray(logits, dtype=np.float32).reshape(-1)
    if capacity < flat.size:
        return -3
    ctypes.memmove(address, flat.ctypes.data, flat.size * 4)
    return 0


def prefill(s: Session, tokens: int, count: int, out_logits: int, capacity: int) -> int:
    if capacity < s._engine.vocab:
        return -3
    return _write(s.prefill(_tokens(tokens, count)), out_logits, capacity)


def decode(s: Session, token: int, out_logits: int, capacity: int) -> int:
    if capacity < s._engine.vocab:
        return -3
    return _write(s.decode(token), out_logits, capacity)


def decode_batch(engine: Ninfer, sessions: List[Session], tokens: int, out_logits: int,
                 capacity: int) -> int:
    if capacity < len(sessions) * engine.vocab:
        return -3
    return _write(engine.decode_batch(sessions, _tokens(tokens, len(sessions))), out_logits,
                  capacity)


def tensor_read(engine: Ninfer, name: str, offset: int, count: int, out: int) -> int:
    return _write(engine.tensor_read(name, offset, count), out, count)


def step(engine: Ninfer, sessions: List[Session], q_len: int, tokens: int, logit_rows: int,
         n_rows: int, out_logits: int, capacity: int) -> int:
    """The C side's flat arrays become (session, tokens, wanted rows) entries."""
    if capacity < n_rows * engine.vocab:
        return -3
    lens = list((ctypes.c_int * len(sessions)).from_address(q_len))
    if min(lens) < 1:
        raise ValueError("ninfer_step: every session brings at least one token")
    flat = _tokens(tokens, sum(lens))
    rows = list((ctypes.c_int * n_rows).from_address(logit_rows)) if n_rows else []
    if rows != sorted(set(rows)) or (rows and not 0 <= rows[0] <= rows[-1] < len(flat)):
        raise ValueError(f"ninfer_step: logit_rows must be ascending rows of the {len(flat)} tokens")
    entries, start = [], 0
    for s, n in zip(sessions, lens):
        entries.append((s, flat[start:start + n], [r - start for r in rows if start <= r < start + n]))
        start += n
    logits = engine.step(entries)
    return 0 if logits is None else _write(logits, out_logits, capacity)


class _Scheduling:
    """The scheduler the C side drives, and its requests by the ids handed out."""

    def __init__(self, engine: Ninfer):
        self.scheduler = Scheduler(engine.runner, engine.sampler)
        self.requests = {}
        self.next_id = 0


def _scheduling(engine: Ninfer) -> _Scheduling:
    if getattr(engine, "_c_scheduling", None) is None:
        engine._c_scheduling = _Scheduling(engine)
    return engine._c_scheduling


def request_add(engine: Ninfer, prompt: int, count: int, max_new_tokens: int, temperature: float,
                top_k: int, top_p: float, repetition_penalty: float, seed: int, stop_ids: int,
                n_stop: int) -> int:
    s = _scheduling(engine)
    params = SamplingParams(temperature, top_k, top_p, repetition_penalty, seed, max_new_tokens)
    rid, s.next_id = s.next_id, s.next_id + 1
    req = Request(str(rid), _tokens(prompt, count), params, _tokens(stop_ids, n_stop) if n_stop else [])
    s.scheduler.add(req)   # (a request that can never run is failed here: request_take says why)
    s.requests[rid] = req
    return rid


def run_step(engine: Ninfer) -> int:
    sched = _scheduling(engine).scheduler
    if sched.has_work():
        sched.step()
    return len(sched.waiting) + len(sched.running)


def request_take(engine: Ninfer, rid: int, out_tokens: int, capacity: int) -> int:
    s = _scheduling(engine)
    sched, requests = s.scheduler, s.requests
    req = requests.get(rid)
    if req is None:
        raise KeyError(f"no request {rid}")
    if not req.done:
        return -4
    if req.status == "failed":
        del requests[rid]
        sched.finished.remove(req)
        raise RuntimeError(f"request {rid} failed: {req.error}")
    if capacity < len(req.output):
        return -3
    if req.output:
        buf = (ctypes.c_longlong * len(req.output))(*req.output)
        ctypes.memmove(out_tokens, buf, 8 * len(req.output))
    del requests[rid]
    sched.finished.remove(req)
    return len(req.output)


def sample(engine: Ninfer, logits: int, temperature: float, top_k: int, top_p: float,
           repetition_penalty: float, seed: int) -> int:
    row = np.ctypeslib.as_array((ctypes.c_float * engine.vocab).from_address(logits))
    return int(engine.sample(row, temperature, top_k, top_p, repetition_penalty, seed))
