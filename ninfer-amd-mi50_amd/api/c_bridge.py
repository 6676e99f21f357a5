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


def sample(engine: Ninfer, logits: int, temperature: float, top_k: int, top_p: float,
           repetition_penalty: float, seed: int) -> int:
    row = np.ctypeslib.as_array((ctypes.c_float * engine.vocab).from_address(logits))
    return int(engine.sample(row, temperature, top_k, top_p, repetition_penalty, seed))
