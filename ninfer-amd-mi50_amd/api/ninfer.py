"""Python entry point in the manner of the reference's ctypes binding
(tools/ninfer_ctypes.py:48-247): a `Ninfer` engine object and `Session`s with
`prefill`, `decode`, `reset`, `close`, `slot`, `length`; `decode_batch` and
`sample` on the engine; the same names and meanings of options where the
reference has them (`max_context`, `prefill_chunk`, `num_sequences`). Logits
come back as numpy arrays. Added for what the reference leaves to an outside
scheduler: `step` (a mixed batch) and `generate` (the scheduler).
Return-code conventions of the C API (src/api/ninfer_c_api.cpp:191,226,235)
become exceptions here.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import numpy as np

from ..config.options import EngineOptions
from ..engine.runner import Chunk
from ..engine.scheduler import Request, Scheduler
from ..loading import load_model, random_model
from ..sampling.params import SamplingParams
from ..sampling.sampler import History, SampleRow, Sampler, fresh_seed


class Session:
    """One request's place in the cache (reference tools/ninfer_ctypes.py:48-90)."""

    def __init__(self, engine: "Ninfer"):
        self._engine = engine
        self._slot: Optional[int] = engine.runner.open()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    @property
    def slot(self) -> int:
        return self._slot

    @property
    def length(self) -> int:
        return self._engine.runner.cache.length(self._slot)

    def reset(self) -> None:
        self._engine.runner.close(self._slot)
        self._slot = self._engine.runner.open()

    def prefill(self, tokens: Sequence[int]) -> np.ndarray:
        """Feed tokens in portions of `prefill_chunk`; logits of the last one
        (reference src/api/ninfer_c_api.cpp:171-198)."""
        if len(tokens) == 0:
            raise ValueError("prefill needs at least one token")
        chunk = self._engine.options.prefill_chunk
        logits = None
        for i in range(0, len(tokens), chunk):
            part = list(tokens[i:i + chunk])
            last = i + chunk >= len(tokens)
            logits = self._engine.runner.step(
                [Chunk(self._slot, part, [len(part) - 1] if last else [])])
        return logits[0].float().cpu().numpy()

    def decode(self, token: int) -> np.ndarray:
        logits = self._engine.runner.step([Chunk(self._slot, [int(token)], [0])])
        return logits[0].float().cpu().numpy()

    def close(self) -> None:
        if self._slot is not None:
            self._engine.runner.close(self._slot)
            self._slot = None


class Ninfer:
    def __init__(self, model_dir: Optional[str] = None, max_context: int = 32768,
                 prefill_chunk: int = 512, num_sequences: int = 1, dtype: str = "bfloat16",
                 page_size: int = 16, num_pages: Optional[int] = None, use_graph: bool = False,
                 random_config: Optional[dict] = None, random_seed: int = 0,
                 random_weights_dtype: Optional[str] = None, kv_bytes: Optional[int] = None,
                 check_pages: bool = False):
        self.options = EngineOptions(dtype=dtype, max_context=max_context,
                                     prefill_chunk=prefill_chunk, num_sequences=num_sequences,
                                     page_size=page_size, num_pages=num_pages,
                                     use_graph=use_graph, kv_bytes=kv_bytes,
                                     check_pages=check_pages)
        if model_dir is not None:
            self.runner = load_model(model_dir, self.options)
        elif random_config is not None:
            self.runner = random_model(random_config, random_seed, self.options,
                                       weights_dtype=random_weights_dtype)
        else:
            raise ValueError("give a model folder or a configuration for random weights")
        self.sampler = Sampler(self.runner.ops, self.runner.device)
        self._sample_calls = 0

    # ---- introspection (reference src/api/ninfer_c_api.h:38-52) --------------------
    @property
    def vocab(self) -> int:
        return self.runner.vocab_size

    @property
    def max_context(self) -> int:
        return self.options.max_context

    @property
    def num_sequences(self) -> int:
        return self.options.num_sequences

    @property
    def devices(self) -> int:
        """GPUs the engine runs on (reference tools/ninfer_ctypes.py:177): always one."""
        return 1

    @property
    def kv_bytes_per_token(self) -> int:
        return self.runner.cache.kv_bytes_per_token(2 if self.options.dtype == "bfloat16" else 4)

    @property
    def state_bytes_per_request(self) -> int:
        """Fixed-size state of a request, apart from its pages (0 for this architecture)."""
        return self.runner.cache.state_bytes_per_request()

    @property
    def kv_total_bytes(self) -> int:
        c = self.runner.cache
        return sum(t.numel() * t.element_size() for pools in c.pools.values()
                   for t in pools.values())

    def kv_pages(self) -> Dict[str, int]:
        c = self.runner.cache
        return {"total": sum(g.allocator.num_pages for g in c.groups),
                "free": sum(g.allocator.free_pages for g in c.groups),
                "reused": c.pages_reused()}

    def tensor_names(self) -> List[str]:
        return self.runner.tensor_names()

    def tensor_read(self, name: str, offset: int = 0, count: Optional[int] = None) -> np.ndarray:
        """`count` numbers (all by default) from flat index `offset` of the checkpoint tensor
        `name` as the engine holds it now, as 32-bit floats: what an outside check needs to
        know of a model whose weights were generated on the device."""
        flat = self.runner.tensor(name).reshape(-1)
        end = flat.numel() if count is None else offset + count
        if not 0 <= offset <= end <= flat.numel():
            raise ValueError(f"{name}: [{offset}, {end}) is outside its {flat.numel()} numbers")
        return flat[offset:end].float().cpu().numpy()

    # ---- sessions -------------------------------------------------------------------
    def session(self) -> Session:
        return Session(self)

    def decode_batch(self, sessions: Sequence[Session], tokens: Sequence[int]) -> np.ndarray:
        """One token for each of several sessions in one step; logits [n, vocab]
        (reference src/api/ninfer_c_api.cpp:219-246)."""
        if len(sessions) != len(tokens):
            raise ValueError("one token per session")
        logits = self.runner.step([Chunk(s.slot, [int(t)], [0])
                                   for s, t in zip(sessions, tokens)])
        return logits.float().cpu().numpy()

    def step(self, entries: Sequence[tuple]) -> Optional[np.ndarray]:
        """A mixed batch: entries of (session, tokens, wanted rows); logits of the
        wanted rows in order, or None."""
        logits = self.runner.step([Chunk(s.slot, list(t), list(w)) for s, t, w in entries])
        return None if logits is None else logits.float().cpu().numpy()

    def sample(self, logits, temperature: float = 0.7, top_k: int = 50, top_p: float = 0.95,
               repetition_penalty: float = 1.0, seed: int = 0,
               recent: Sequence[int] = ()) -> int:
        """Stateless sampling of one row (reference src/api/ninfer_c_api.cpp:248-260;
        there the history is empty, here `recent` may carry it)."""
        import torch
        row = torch.as_tensor(np.asarray(logits, dtype=np.float32)).reshape(1, -1).to(
            self.runner.device)
        params = SamplingParams(temperature, top_k, top_p, repetition_penalty, seed, 1)
        self._sample_calls += 1
        r = SampleRow(params, History(recent), 0, 0 if seed else self._sample_calls,
                      seed or fresh_seed())
        return self.sampler.sample(row, [r])[0]

    def close(self) -> None:
        """Give the model, its cache, its captured graphs and the kernels' workspaces back to
        the device (reference tools/ninfer_ctypes.py:238-241: ninfer_free); the object cannot
        be used afterwards. After it another engine may take this one's place in memory."""
        import gc
        import torch
        if self.runner is not None:
            self.runner.release()
        self.runner = None
        self.sampler = None
        gc.collect()
        if torch.cuda.is_available():
            torch.cuda.synchronize()
            torch.cuda.empty_cache()

    # ---- generation -----------------------------------------------------------------
    def generate(self, prompts: Sequence[Sequence[int]], params: Optional[SamplingParams] = None,
                 stop_ids: Optional[Sequence[int]] = None) -> List[List[int]]:
        """Generated token ids for each prompt, through the scheduler."""
        params = params or SamplingParams()
        if stop_ids is None:
            stop_ids = list(self.runner.spec.eos_token_ids)
        sched = Scheduler(self.runner, self.sampler)
        reqs = [Request(str(i), list(p), params, stop_ids) for i, p in enumerate(prompts)]
        for r in reqs:
            sched.add(r)
        sched.run()
        for r in reqs:
            if r.status == "failed":
                raise RuntimeError(f"request {r.id}: {r.error}")
        return [r.output for r in reqs]
