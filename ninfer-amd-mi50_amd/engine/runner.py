"""The step function: one batch of (request, its next tokens) through the
model, from the cache, to logits at the wanted rows.

A batch may hold portions of prompts beside single decoded tokens, cut
anywhere. Only the tokens given are run; everything earlier comes from the
cache. The reference's counterpart is `Model::forward_batch`
(src/models/model.hip:994-1065): rows = (token, position, sequence slot),
groups = runs of equal slots (:950-961), logits for the last row of each group
only (:727-755), and a host sync per sparse layer (src/ops/moe.hip:53). Here
positions come from the cache manager, logits are returned for any asked
rows, and nothing inside a step waits for the device.
"""
from __future__ import annotations

from collections import OrderedDict
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch

from ..cache.manager import CacheManager
from ..config.options import EngineOptions
from ..models.spec import ModelSpec
from ..parts.base import CacheView, CallInfo, StepContext, WeightBinder
from ..weights.source import check_tensors

_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32}


@dataclass
class Chunk:
    """The next tokens of one request in a step and the rows (indices into
    `tokens`) whose logits are wanted."""
    slot: int
    tokens: Sequence[int]
    want: Sequence[int] = field(default_factory=list)


class ModelRunner:
    """Owns the bound model, the cache manager and the step function."""

    def __init__(self, spec: ModelSpec, source, options: EngineOptions, ops=None,
                 where: str = "model"):
        options.validate()
        self.spec = spec
        self.options = options
        self.device = torch.device(options.device)
        self.act_dtype = _DTYPES[options.dtype]
        if ops is None:
            from ..kernels import load_ops
            ops = load_ops()
        self.ops = ops
        limit = spec.max_positions()
        if limit is not None and options.max_context > limit:
            raise ValueError(f"max_context {options.max_context} is beyond the {limit} positions "
                             f"that the model's parts allow")
        check_tensors(source.shapes(), spec.tensor_specs(), where, spec.unused_tensor_specs())
        binder = WeightBinder(source, self.device, self.act_dtype)
        spec.bind(binder)
        self._held = binder.held

        # one cache instance per plan entry that writes keys and values
        needs = []
        self._state_range: List[Optional[slice]] = []
        floats = 0
        for call in spec.plan:
            mixer = spec.blocks[call.layer].mixer
            needs.append(mixer.cache_need() if call.cache_from is None else None)
            n = mixer.state_floats()
            self._state_range.append(slice(floats, floats + n) if n else None)
            floats += n
        own = {"float32": 4, "bfloat16": 2}
        per_token = sum(p.elements_per_token() * own[p.dtype or options.dtype]
                        for n in needs if n is not None for p in n.pools)
        self.cache = CacheManager(needs, options.page_size, options.pool_pages(per_token),
                                  options.num_sequences, options.max_context, floats)
        for g in self.cache.groups:
            if g.page_size != options.page_size:   # a mixer's own page size: the same warning
                options.warn_of_slow_pages(g.page_size)
        self.cache.allocate_pools(self.device, self.act_dtype, ops=self.ops)
        self.cache.poison_freed = options.poison_freed_pages
        self.vocab_size = spec.vocab_size
        self.steps_run = 0
        # captured decode steps by (requests, context bound), least recently replayed first;
        # at most options.max_graphs are kept (each holds a memory pool of its own)
        self._graphs: "OrderedDict[tuple, dict]" = OrderedDict()
        self.graphs_dropped = 0
        self._holds_graphs = False
        self.graph_context_step = 1024   # a graph serves contexts up to the next multiple

    # ---- read-back -------------------------------------------------------------
    def tensor_names(self) -> List[str]:
        return sorted(self._held)

    def tensor(self, name: str) -> torch.Tensor:
        """The checkpoint tensor `name` as the engine holds it now: a view of the
        device memory its kernels read (a slice of a fused or stacked tensor
        where parts fuse), in the dtype it is kept in. For tests and tools that
        have to know what a model generated on the device holds."""
        if name not in self._held:
            raise KeyError(f"the model holds no tensor named {name!r}")
        return self._held[name]

    # ---- requests --------------------------------------------------------------
    def open(self) -> int:
        return self.cache.acquire()

    def close(self, slot: int) -> None:
        self.cache.release(slot)

    def release(self) -> None:
        """Drop everything this runner holds on the device: captured graphs (and with them
        their memory pools), staging buffers, the cache's pools, the bound weights. The
        kernels' workspaces go too once no runner with captured graphs is left. The runner
        cannot step afterwards."""
        self._graphs.clear()
        if self._holds_graphs:
            self._holds_graphs = False
            self.ops.graph_holder_gone(self)
        self._staging = []
        self._held = {}
        self.cache.drop_pools()
        self.spec = None

    # ---- the step ----------------------------------------------------------------
    def step(self, chunks: Sequence[Chunk]) -> Optional[torch.Tensor]:
        """Run one batch. Returns 32-bit logits [R, vocab] on the device for
        the wanted rows, in the order of the chunks and of their `want`, or
        None if none are wanted. Raises OutOfPages (nothing run, nothing
        reserved beyond what fits) when pages do not suffice."""
        if not chunks:
            return None
        cache = self.cache
        for c in chunks:
            if len(c.tokens) < 1:
                raise ValueError("a request in a step brings at least one token")
        # Requests that bring one token go first (a stable sort), so that their rows are the
        # step's first: attention then runs them apart from the prompt portions. The wanted
        # rows keep the order of the caller's chunks.
        given = chunks
        chunks = sorted(given, key=lambda c: len(c.tokens) != 1)
        single_rows = sum(1 for c in chunks if len(c.tokens) == 1)
        slots = [c.slot for c in chunks]
        if len(set(slots)) != len(slots):
            raise ValueError("a request may appear once in a step")
        pos0 = [cache.length(c.slot) for c in chunks]
        T = sum(len(c.tokens) for c in chunks)
        S = len(chunks)
        tokens = np.empty(T, np.int32)
        positions = np.empty(T, np.int32)
        row_seq = np.empty(T, np.int32)
        row_start = np.empty(S + 1, np.int32)
        qlen = np.empty(S, np.int32)
        first_row = {}
        r = 0
        for i, (c, p) in enumerate(zip(chunks, pos0)):
            n = len(c.tokens)
            tokens[r:r + n] = np.asarray(c.tokens, dtype=np.int64)
            positions[r:r + n] = np.arange(p, p + n)
            row_seq[r:r + n] = i
            row_start[i] = r
            qlen[i] = n
            first_row[c.slot] = r
            r += n
        row_start[S] = T
        want_rows: List[int] = []
        for c in given:
            for w in c.want:
                if not 0 <= w < len(c.tokens):
                    raise ValueError(f"wanted row {w} is outside the request's "
                                     f"{len(c.tokens)} tokens")
                want_rows.append(first_row[c.slot] + w)
        if tokens.min() < 0 or tokens.max() >= self.vocab_size:
            raise ValueError(f"token id outside [0, {self.vocab_size})")
        # the batch is well formed: now pages for all its requests, or for none
        cache.reserve_all([(c.slot, p + len(c.tokens)) for c, p in zip(chunks, pos0)])
        max_kv_len = int(max(p + len(c.tokens) for c, p in zip(chunks, pos0)))
        graph = (self.options.use_graph and self.device.type == "cuda" and int(qlen.max()) == 1
                 and want_rows == list(range(T)))
        # a graph is replayed for many steps: fixed table width, context rounded up
        if graph:
            max_kv_len = min(-(-max_kv_len // self.graph_context_step) * self.graph_context_step,
                             min(g.max_pages * g.page_size for g in cache.groups)
                             if cache.groups else cache.max_pages_per_request * cache.page_size)
        tables = [cache.block_table(g, slots, cache.groups[g].max_pages if graph else None)
                  for g in range(len(cache.groups))]
        if self.options.check_pages:
            self._check_pages(chunks, pos0, tables)
        parts = [tokens, positions, row_seq, np.asarray(slots, np.int32), row_start, qlen,
                 np.asarray(pos0, np.int32), np.asarray(want_rows, np.int32)]
        parts += [t.reshape(-1) for t in tables]
        sizes = [x.size for x in parts]
        host = torch.from_numpy(np.concatenate(parts))
        shape = dict(T=T, S=S, sizes=sizes, widths=[t.shape[1] for t in tables],
                     max_qlen=int(qlen.max()), max_kv_len=max_kv_len, wants=bool(want_rows),
                     single_rows=single_rows)
        if graph:
            logits = self._step_graph(host, shape)
        else:
            logits = self._forward(self._to_device(host), shape)
        for c, p in zip(chunks, pos0):
            cache.commit(c.slot, p + len(c.tokens))
        self.steps_run += 1
        return logits

    def _to_device(self, host: torch.Tensor) -> torch.Tensor:
        """The step's packed index buffer on the device, copied through one of a few pinned
        staging buffers that are kept and used in turn (allocating pinned memory every step
        costs more than the copy). A buffer is reused only after the copy out of it has run."""
        if self.device.type != "cuda":
            return host
        n = host.numel()
        if not hasattr(self, "_staging"):
            self._staging, self._staging_next = [], 0
        if len(self._staging) < 4:
            self._staging.append([torch.empty(max(n, 4096), dtype=torch.int32).pin_memory(),
                                  torch.cuda.Event()])
            slot = self._staging[-1]
        else:
            slot = self._staging[self._staging_next]
            self._staging_next = (self._staging_next + 1) % len(self._staging)
            slot[1].synchronize()
            if slot[0].numel() < n:
                slot[0] = torch.empty(2 * n, dtype=torch.int32).pin_memory()
        slot[0][:n].copy_(host)
        dev = torch.empty(n, dtype=torch.int32, device=self.device)
        dev.copy_(slot[0][:n], non_blocking=True)
        slot[1].record()
        return dev

    def _check_pages(self, chunks: Sequence[Chunk], pos0: List[int], tables) -> None:
        """Debugging: what the kernels assume of the step's block tables, checked on the host
        before anything is launched. Every entry is -1 or a page of the pool; every position
        the step writes, and every earlier one its rows can see, lies in a page that the
        allocator counts as held; no page stands in two requests' rows. (The reference's
        analogue is the overflow throw of its slab, src/runtime/kv_cache.cpp:35-37.)"""
        for g, table in zip(self.cache.groups, tables):
            ps = g.page_size
            owner: Dict[int, int] = {}
            for i, (c, p) in enumerate(zip(chunks, pos0)):
                row = table[i]
                if ((row < -1) | (row >= g.allocator.num_pages)).any():
                    raise RuntimeError(f"slot {c.slot}: block table holds a page outside "
                                       f"[0, {g.allocator.num_pages}): {row.tolist()}")
                lo = 0 if g.window is None else max(0, p - g.window + 1)
                last = p + len(c.tokens) - 1
                if last // ps >= row.shape[0]:
                    raise RuntimeError(f"slot {c.slot}: position {last} is beyond the block "
                                       f"table's {row.shape[0]} pages")
                for lp in range(lo // ps, last // ps + 1):
                    page = int(row[lp])
                    if page < 0 or not g.allocator.is_held(page):
                        raise RuntimeError(f"slot {c.slot}: positions {lp * ps}.. are read or "
                                           f"written, but page {page} is not held")
                for page in row[row >= 0].tolist():
                    if owner.setdefault(page, c.slot) != c.slot:
                        raise RuntimeError(f"page {page} stands in the block tables of slots "
                                           f"{owner[page]} and {c.slot}")

    def _forward(self, dev: torch.Tensor, shape: dict) -> Optional[torch.Tensor]:
        """Run the model on the step described by the packed index buffer `dev`
        (tokens, positions, row_seq, slots, row_start, qlen, pos0, wanted rows,
        then one block table per cache group)."""
        views = []
        o = 0
        for n in shape["sizes"]:
            views.append(dev[o:o + n])
            o += n
        S = shape["S"]
        d_tables = [v.view(S, w) for v, w in zip(views[8:], shape["widths"])]
        ctx = StepContext(
            ops=self.ops, act_dtype=self.act_dtype, device=self.device, T=shape["T"], S=S,
            tokens=views[0], positions=views[1], row_seq=views[2], seq_slots=views[3],
            seq_row_start=views[4], seq_qlen=views[5], seq_pos0=views[6],
            max_qlen=shape["max_qlen"], max_kv_len=shape["max_kv_len"],
            all_decode=shape["max_qlen"] == 1, single_rows=shape["single_rows"])
        return self.spec.forward(ctx, self._call_infos(d_tables),
                                 views[7] if shape["wants"] else None)

    def _step_graph(self, host: torch.Tensor, shape: dict) -> torch.Tensor:
        """Decode-only steps replayed from a captured HIP graph: one graph per
        (requests in the step, context bound). The index buffer is the graph's
        only input; it is refreshed by one copy before every replay. The first
        step of a shape runs eagerly (it also sizes every workspace), the
        second is captured. The reference captures its single-token dense
        decode the same way (src/models/model.hip:786-830). The returned logits
        live in the graph's memory and are valid until the next step."""
        key = (shape["S"], shape["max_kv_len"])
        entry = self._graphs.get(key)
        if entry is not None:
            self._graphs.move_to_end(key)
        if entry is None:
            # The least recently replayed graphs make room. Logits handed out by a dropped
            # graph were valid until this step only, as those of every graph are; the entry's
            # own reference to them goes with it, and the pool's memory returns to the
            # allocator once the caller's last reference is gone.
            while len(self._graphs) >= max(1, self.options.max_graphs):
                self._graphs.popitem(last=False)
                self.graphs_dropped += 1
            self._graphs[key] = {"pinned": torch.empty(host.numel(), dtype=torch.int32).pin_memory(),
                                 "meta": torch.empty(host.numel(), dtype=torch.int32,
                                                     device=self.device), "graph": None}
            entry = self._graphs[key]
            entry["copied"] = torch.cuda.Event()
            entry["pinned"].copy_(host)
            entry["meta"].copy_(entry["pinned"], non_blocking=True)
            entry["copied"].record()
            return self._forward(entry["meta"], shape)
        # the pinned staging buffer is reused: wait until the last copy from it is done (a
        # caller that does not read the logits of a step back runs ahead of the device)
        entry["copied"].synchronize()
        entry["pinned"].copy_(host)
        entry["meta"].copy_(entry["pinned"], non_blocking=True)
        entry["copied"].record()
        if entry["graph"] is None:
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                entry["logits"] = self._forward(entry["meta"], shape)
            entry["graph"] = g
            if not self._holds_graphs:
                self._holds_graphs = True
                self.ops.graph_holder_new(self)
        entry["graph"].replay()
        return entry["logits"]

    def _call_infos(self, d_tables: List[torch.Tensor]) -> List[CallInfo]:
        cache = self.cache
        infos = []
        for i, call in enumerate(self.spec.plan):
            owner = i if call.cache_from is None else call.cache_from
            view = None
            if owner in cache.pools:
                g = cache.group_of_instance[owner]
                view = CacheView(cache.pools[owner], d_tables[g], cache.groups[g].page_size,
                                 cache.groups[g].window)
            rng = self._state_range[i]
            state = cache.state[:, rng] if rng is not None else None
            infos.append(CallInfo(cache=view, writes_cache=call.cache_from is None, state=state))
        return infos
