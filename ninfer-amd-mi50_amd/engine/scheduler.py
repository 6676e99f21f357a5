"""The scheduler above the step function: admits requests, cuts prompts into
portions under a token budget, decodes, finishes and frees.

The reference has no scheduler in the engine: `Engine::run` serves one request
at a time with fixed `prefill_chunk` portions (src/runtime/engine.cpp:122-205),
finishes on a special token or `max_new_tokens` (:156, :173), rejects a prompt
that cannot fit (:124-127) and throws when its slab overflows
(src/runtime/kv_cache.cpp:35-37); batching is left to an outside scheduler.

Every step is built in this order, under `max_batch_tokens` and `max_seqs`:
 1. one decode token for every running request whose prompt is in the cache;
 2. the next portion min(remaining, budget left) of running requests still in
    their prompt, oldest first;
 3. requests from the waiting queue (first in, first out) while a slot is
    free, budget is left and the pages of the first portion can be had.
Logits are asked for decode rows and for the portion that ends a prompt.

When pages run out: a decode token or portion that cannot get its pages
preempts the most recently admitted running request (its pages and slot are
given back, it returns to the front of the waiting queue and later recomputes
prompt + generated tokens). Only requests that arrived after the one in need
are preempted for it: an older request is never given back for a newer one,
which waits instead (it brings no tokens to this step). A request that could
not fit even alone is finished with an error; in a group of windowed layers
"fit" means the window plus one step's portion, since older pages are given
back as the window passes them.
"""
from __future__ import annotations

import hashlib
from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Dict, List, Optional, Sequence, Tuple

from ..cache.pages import OutOfPages
from ..sampling.params import SamplingParams
from ..sampling.sampler import History, SampleRow, fresh_seed
from .runner import Chunk


@dataclass
class Request:
    id: str
    prompt: List[int]
    params: SamplingParams = field(default_factory=SamplingParams)
    stop_ids: Sequence[int] = ()
    # progress
    output: List[int] = field(default_factory=list)
    slot: Optional[int] = None
    cached: int = 0                 # tokens of prompt + output that are in the cache
    status: str = "waiting"         # waiting | running | finished | failed
    error: Optional[str] = None
    preemptions: int = 0
    seed: int = 0
    key: int = 0                    # of its stream of random numbers: from its id (see add)
    order: int = 0                  # of its arrival at the scheduler
    history: History = field(default_factory=History)

    @property
    def tokens(self) -> List[int]:
        return self.prompt + self.output

    @property
    def done(self) -> bool:
        return self.status in ("finished", "failed")

    def next_tokens(self, n: int) -> List[int]:
        """The n tokens after the cached ones (without joining prompt and output)."""
        a, b, p = self.cached, self.cached + n, len(self.prompt)
        if b <= p:
            return self.prompt[a:b]
        if a >= p:
            return self.output[a - p:b - p]
        return self.prompt[a:] + self.output[:b - p]


@dataclass
class PlannedStep:
    chunks: List[Tuple[Request, int, bool]]   # (request, tokens to feed, wants logits)
    preempted: List[Request]
    failed: List[Request]


class Scheduler:
    def __init__(self, runner, sampler, max_batch_tokens: Optional[int] = None,
                 max_seqs: Optional[int] = None):
        self.runner = runner
        self.cache = runner.cache
        self.sampler = sampler
        self.max_batch_tokens = max_batch_tokens or runner.options.prefill_chunk
        self.max_seqs = max_seqs or runner.options.num_sequences
        self.waiting: Deque[Request] = deque()
        self.running: List[Request] = []      # in order of admission
        self.finished: List[Request] = []
        self._next_key = 0
        self.steps = 0
        self.preemptions = 0

    # ---- requests ----------------------------------------------------------------
    def add(self, request: Request) -> None:
        if not request.prompt:
            request.status, request.error = "failed", "empty prompt"
            self.finished.append(request)
            return
        if len(request.prompt) + request.params.max_new_tokens > self.cache.max_context:
            # the reference's rule (src/runtime/engine.cpp:124-127)
            request.status = "failed"
            request.error = "prompt + max_new_tokens exceeds max_context"
            self.finished.append(request)
            return
        request.seed = request.params.seed if request.params.seed != 0 else fresh_seed()
        # The stream of random numbers is named by (seed, id), not by the order of arrival:
        # the same request draws the same tokens alone and in a crowd, and requests that
        # share a seed still draw differently.
        digest = hashlib.sha256(str(request.id).encode("utf-8")).digest()
        request.key = int.from_bytes(digest[:8], "little")
        request.order = self._next_key
        self._next_key += 1
        request.history = History(request.prompt)
        request.status = "waiting"
        self.waiting.append(request)

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    # ---- planning (host only) ------------------------------------------------------
    def _pages_for(self, req: Request, n: int) -> List[int]:
        return self.cache.pages_needed(req.slot, req.cached + n)

    def _fits_alone(self, total: int) -> bool:
        """Could a request of `total` tokens run with every page to itself? A group that
        keeps all keys must hold them all; a windowed group never holds more than the span a
        step of n tokens touches, the window - 1 keys before its first row and its n rows
        (pages the window has passed are given back after every step): window + n - 1
        positions, which lie in at most ceil(that / page) + 1 pages wherever they start."""
        for g in self.cache.groups:
            ps = g.page_size
            most = -(-total // ps)
            if g.window is not None:
                most = min(most, -(-(g.window + self.max_batch_tokens - 1) // ps) + 1)
            if most > g.allocator.num_pages:
                return False
        return True

    def plan(self) -> PlannedStep:
        """Decide the next step. Acquires slots for admitted requests and
        releases preempted ones; touches no pages."""
        cache = self.cache
        budget = self.max_batch_tokens
        free = [g.allocator.free_pages for g in cache.groups]
        chunks: List[Tuple[Request, int, bool]] = []
        preempted: List[Request] = []
        failed: List[Request] = []

        def take(req: Request, n: int) -> bool:
            need = self._pages_for(req, n)
            if any(a > b for a, b in zip(need, free)):
                return False
            for i, a in enumerate(need):
                free[i] -= a
            return True

        def preempt_newest(keep: Request) -> bool:
            """Give back the newest running request that arrived after `keep`
            and is not yet part of this step; false if there is none."""
            planned = {id(c[0]) for c in chunks}
            for victim in sorted(self.running, key=lambda r: -r.order):
                if victim is keep or id(victim) in planned or victim.order < keep.order:
                    continue
                for i, g in enumerate(cache.groups):
                    free[i] += sum(1 for p in g.tables[victim.slot] if p >= 0)
                cache.release(victim.slot)
                victim.slot, victim.cached, victim.status = None, 0, "waiting"
                victim.preemptions += 1
                self.preemptions += 1
                self.running.remove(victim)
                preempted.append(victim)
                return True
            return False

        # 1 and 2: running requests, oldest first; decode tokens before portions
        order = [r for r in self.running if r.cached >= len(r.prompt)] + \
                [r for r in self.running if r.cached < len(r.prompt)]
        for req in order:
            if req not in self.running or budget <= 0:
                continue
            left = len(req.tokens) - req.cached
            n = min(left, budget)
            while not take(req, n):
                if not preempt_newest(req):
                    n = 0
                    break
            if n == 0:
                if len(self.running) == 1 and not chunks:
                    # alone and still no room: it can never fit
                    cache.release(req.slot)
                    self.running.remove(req)
                    req.slot, req.status = None, "failed"
                    req.error = "the request does not fit in the cache"
                    failed.append(req)
                continue
            chunks.append((req, n, n == left))
            budget -= n
        # preempted requests go back to the front, oldest first
        for req in sorted(preempted, key=lambda r: -r.order):
            self.waiting.appendleft(req)
        # 3: admissions
        while self.waiting and budget > 0 and len(self.running) < self.max_seqs \
                and cache.free_slots > 0 and not preempted:
            req = self.waiting[0]
            total = len(req.tokens)
            if total > cache.max_context or not self._fits_alone(total):
                self.waiting.popleft()
                req.status, req.error = "failed", "the request does not fit in the cache"
                failed.append(req)
                continue
            n = min(total, budget)
            req.slot = cache.acquire()
            if not take(req, n):
                cache.release(req.slot)
                req.slot = None
                break
            self.waiting.popleft()
            req.status = "running"
            self.running.append(req)
            chunks.append((req, n, n == total))
            budget -= n
        self.finished.extend(failed)
        return PlannedStep(chunks, preempted, failed)

    # ---- one step --------------------------------------------------------------------
    def step(self) -> List[Request]:
        """Plan, run and sample one step; returns the requests it finished."""
        planned = self.plan()
        done: List[Request] = list(planned.failed)
        if not planned.chunks:
            if self.has_work() and not planned.failed and not planned.preempted:
                raise RuntimeError("scheduler made no progress")
            return done
        chunks = []
        for req, n, want in planned.chunks:
            chunks.append(Chunk(req.slot, req.next_tokens(n), [n - 1] if want else []))
        logits = self.runner.step(chunks)
        self.steps += 1
        rows = []
        wanting = []
        for req, n, want in planned.chunks:
            req.cached += n
            if want:
                wanting.append(req)
                rows.append(SampleRow(req.params, req.history, req.key, len(req.output), req.seed))
        if wanting:
            tokens = self.sampler.sample(logits, rows)
            for req, tok in zip(wanting, tokens):
                if tok in req.stop_ids:
                    self._finish(req)            # the stop token is not part of the output
                    done.append(req)
                    continue
                req.output.append(tok)
                req.history.add(tok)
                if len(req.output) >= req.params.max_new_tokens:
                    self._finish(req)
                    done.append(req)
        return done

    def _finish(self, req: Request) -> None:
        self.cache.release(req.slot)
        req.slot, req.status = None, "finished"
        self.running.remove(req)
        self.finished.append(req)

    def run(self) -> List[Request]:
        """Steps until every request is finished."""
        while self.has_work():
            self.step()
        return self.finished
