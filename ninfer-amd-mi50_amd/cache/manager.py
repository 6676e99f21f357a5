"""Cache manager: paged keys and values with a block table per request, and
slots of fixed-size per-request state.

Layers whose mixers need the same span of the past, in pages of the same size, form
a *group*: all keys (window None) or the last `window` positions; the engine's page
size or one the mixer asks for. A group has its own page ids,
allocator and block tables; every cache instance (one per plan entry that
writes keys and values) in the group has its own pools (any number, named,
each with a per-token shape and dtype of its own), indexed by the group's
page ids. A request holds one *slot*: its row in every group's block
table and its row of the state tensor.

Pages are given back when a request is released and, in a window group, as
soon as the window has passed them: with n cached positions, the next query
is at position >= n and sees keys >= n - window + 1, so every page whose last
position is <= n - window is freed (its block-table entry becomes -1).

The reference's cache is one slab per (layer, slot) addressed by
seq * stride + pos * Hkv * D (src/runtime/kv_cache.h:25-42); its lengths live
in the caller (src/api/ninfer_c_api.cpp:28-32). Introspection successors of
src/api/ninfer_c_api.cpp:99-114: `kv_bytes_per_token`, `pages_total`,
`pages_free`.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

from ..parts.base import CacheNeed
from .pages import OutOfPages, PageAllocator


@dataclass
class CacheGroup:
    window: Optional[int]
    allocator: PageAllocator
    page_size: int = 0                                    # tokens a page of this group holds
    max_pages: int = 0                                    # pages a request can hold at most
    instances: List[int] = field(default_factory=list)   # plan entries with pools in this group
    tables: Dict[int, List[int]] = field(default_factory=dict)  # slot -> page of each logical page
    window_freed: int = 0
    # the same tables as rows of one array [slots, pages a request can hold], -1 where no page
    # is held: what a step copies its block table from
    rows: Optional[np.ndarray] = None


class CacheManager:
    """Host side of the cache: who holds which page. Device pools are made by
    `allocate_pools` so that this class can be tested without a device."""

    def __init__(self, needs: Sequence[Optional[CacheNeed]], page_size: int, num_pages: int,
                 max_seqs: int, max_context: int, state_floats: int = 0):
        self.page_size = page_size
        self.max_seqs = max_seqs
        self.max_context = max_context
        self.max_pages_per_request = -(-max_context // page_size)
        self.state_floats = state_floats
        self.needs = list(needs)
        self.groups: List[CacheGroup] = []
        self.group_of_instance: Dict[int, int] = {}
        by_kind: Dict[Tuple[Optional[int], int], int] = {}
        for i, need in enumerate(self.needs):
            if need is None:
                continue
            ps = need.page_size if need.page_size is not None else page_size
            if ps < 1:
                raise ValueError(f"a mixer asks for pages of {ps} tokens")
            if (need.window, ps) not in by_kind:
                by_kind[(need.window, ps)] = len(self.groups)
                # `num_pages` counts pages of the engine's size: a group with pages of another
                # size gets as many as hold the same number of tokens
                n = num_pages if ps == page_size else max(1, num_pages * page_size // ps)
                self.groups.append(CacheGroup(need.window, PageAllocator(n), page_size=ps,
                                              max_pages=-(-max_context // ps)))
            g = by_kind[(need.window, ps)]
            self.groups[g].instances.append(i)
            self.group_of_instance[i] = g
        for g in self.groups:
            g.rows = np.full((max_seqs, g.max_pages), -1, dtype=np.int32)
        self._free_slots: List[int] = list(range(max_seqs - 1, -1, -1))
        self._length: Dict[int, int] = {}
        self.pools: Dict[int, Dict[str, object]] = {}   # cache instance -> pool name -> tensor
        self.state = None
        # debugging: pages given back are filled with NaN in every pool of their group, so
        # that a read of a page that is no longer held (or of a slot not yet written in a page
        # that is used again) shows in the logits
        self.poison_freed = False

    # ---- device memory -----------------------------------------------------
    def allocate_pools(self, device, dtype, ops=None) -> None:
        """Device memory of every pool, [pages, *outer, page_size, *inner] in the pool's own
        dtype (the activation dtype `dtype` where it names none), and the state tensor.
        `ops` (the kernel library) fills freed pages with NaN when poisoning is on."""
        import torch
        self._ops = ops
        named = {"float32": torch.float32, "bfloat16": torch.bfloat16}
        for i, need in enumerate(self.needs):
            if need is None:
                continue
            group = self.groups[self.group_of_instance[i]]
            n = group.allocator.num_pages
            self.pools[i] = {}
            for spec in need.pools:
                if spec.name in self.pools[i]:
                    raise ValueError(f"a mixer names two pools {spec.name!r}")
                if spec.dtype is not None and spec.dtype not in named:
                    raise ValueError(f"pool {spec.name!r}: dtype {spec.dtype!r} is not one of "
                                     f"{sorted(named)}")
                shape = (n, *spec.outer, group.page_size, *spec.inner)
                self.pools[i][spec.name] = torch.zeros(
                    shape, dtype=named[spec.dtype] if spec.dtype else dtype, device=device)
        self.state = torch.zeros((self.max_seqs, max(self.state_floats, 1)),
                                 dtype=torch.float32, device=device)

    def drop_pools(self) -> None:
        """Give the device memory of every pool and of the state back (the end of an engine)."""
        self.pools = {}
        self.state = None

    # ---- slots ---------------------------------------------------------------
    @property
    def free_slots(self) -> int:
        return len(self._free_slots)

    def live_slots(self) -> List[int]:
        return sorted(self._length)

    def acquire(self) -> int:
        """A free slot with empty block tables and zeroed state."""
        if not self._free_slots:
            raise RuntimeError(f"all {self.max_seqs} request slots are in use")
        slot = self._free_slots.pop()
        self._length[slot] = 0
        for g in self.groups:
            g.tables[slot] = []
            g.rows[slot, :] = -1
        if self.state is not None and self.state_floats:
            self.state[slot].zero_()
        return slot

    def release(self, slot: int) -> None:
        """Give back every page the request holds in every group, and its slot."""
        if slot not in self._length:
            raise RuntimeError(f"slot {slot} released but not held")
        for g in self.groups:
            self._give_back(g, [p for p in g.tables.pop(slot) if p >= 0])
        del self._length[slot]
        self._free_slots.append(slot)

    def _give_back(self, g: CacheGroup, pages: List[int]) -> None:
        g.allocator.free(pages)
        if self.poison_freed and pages and self.pools:
            import torch
            for i in g.instances:
                for pool in self.pools[i].values():
                    idx = torch.tensor(pages, dtype=torch.int32, device=pool.device)
                    if getattr(self, "_ops", None) is not None:
                        self._ops.fill_nan_pages(pool, idx)
                    else:   # no kernel library (host tests)
                        pool.index_fill_(0, idx.long(), float("nan"))

    def length(self, slot: int) -> int:
        return self._length[slot]

    # ---- pages ---------------------------------------------------------------
    def pages_needed(self, slot: int, new_len: int) -> List[int]:
        return [max(0, -(-new_len // g.page_size) - len(g.tables[slot])) for g in self.groups]

    def can_reserve(self, slot: int, new_len: int) -> bool:
        return all(n <= g.allocator.free_pages
                   for n, g in zip(self.pages_needed(slot, new_len), self.groups))

    def reserve(self, slot: int, new_len: int) -> None:
        """Pages for positions < new_len in every group, or OutOfPages with
        nothing taken in any group."""
        if new_len > self.max_context:
            raise OutOfPages(f"request would hold {new_len} tokens; max_context is "
                             f"{self.max_context}")
        need = self.pages_needed(slot, new_len)
        for n, g in zip(need, self.groups):
            if n > g.allocator.free_pages:
                raise OutOfPages(f"need {n} pages in the group with window {g.window}, "
                                 f"{g.allocator.free_pages} are free")
        for n, g in zip(need, self.groups):
            if n:
                table = g.tables[slot]
                pages = g.allocator.alloc(n)
                g.rows[slot, len(table):len(table) + n] = pages
                table.extend(pages)

    def reserve_all(self, wants: Sequence[Tuple[int, int]]) -> None:
        """`reserve` for several (slot, new_len) at once: all or nothing."""
        total = [0] * len(self.groups)
        for slot, new_len in wants:
            if new_len > self.max_context:
                raise OutOfPages(f"request would hold {new_len} tokens; max_context is "
                                 f"{self.max_context}")
            for i, n in enumerate(self.pages_needed(slot, new_len)):
                total[i] += n
        for n, g in zip(total, self.groups):
            if n > g.allocator.free_pages:
                raise OutOfPages(f"need {n} pages in the group with window {g.window}, "
                                 f"{g.allocator.free_pages} are free")
        for slot, new_len in wants:
            self.reserve(slot, new_len)

    def commit(self, slot: int, new_len: int) -> None:
        """The request now has new_len cached positions; free what its windows
        have passed."""
        if new_len < self._length[slot]:
            raise RuntimeError("a request's cached length cannot shrink")
        self._length[slot] = new_len
        for g in self.groups:
            if g.window is None:
                continue
            table = g.tables[slot]
            # pages whose last position (p+1)*ps - 1 <= new_len - window
            dead = (new_len - g.window + 1) // g.page_size
            gone = []
            for p in range(min(max(dead, 0), len(table))):
                if table[p] >= 0:
                    gone.append(table[p])
                    table[p] = -1
                    g.rows[slot, p] = -1
            if gone:
                self._give_back(g, gone)
                g.window_freed += len(gone)

    # ---- what a step needs ---------------------------------------------------
    def block_table(self, group: int, slots: Sequence[int], width: Optional[int] = None
                    ) -> np.ndarray:
        """int32 [len(slots), width] block-table rows, -1 where no page is held."""
        g = self.groups[group]
        if width is None:
            width = max([len(g.tables[s]) for s in slots] + [1])
        return g.rows[np.asarray(slots, dtype=np.intp), :width]   # a copy

    # ---- introspection -------------------------------------------------------
    def state_bytes_per_request(self) -> int:
        """Bytes of fixed-size state a request holds whatever its length (32-bit floats of every
        mixer that keeps such state): reported apart from the pages' bytes per token, so that
        whoever sizes the cache can count both."""
        return 4 * self.state_floats

    def kv_bytes_per_token(self, bytes_per_element: int) -> int:
        """Bytes of paged cache one token takes over all cache instances; pools without a
        dtype of their own count `bytes_per_element` per number."""
        own = {"float32": 4, "bfloat16": 2}
        return sum(p.elements_per_token() * (own[p.dtype] if p.dtype else bytes_per_element)
                   for n in self.needs if n is not None for p in n.pools)

    def pages_total(self, group: int = 0) -> int:
        return self.groups[group].allocator.num_pages

    def pages_free(self, group: int = 0) -> int:
        return self.groups[group].allocator.free_pages

    def pages_reused(self) -> int:
        return sum(g.allocator.reused for g in self.groups)

    def check(self) -> None:
        """No page lost, held twice, or held by nobody."""
        for g in self.groups:
            g.allocator.check()
            held = [p for t in g.tables.values() for p in t if p >= 0]
            assert len(held) == len(set(held)), "a page is in two block tables"
            assert len(held) == g.allocator.in_use, "allocator and block tables disagree"
            for slot, t in g.tables.items():
                assert g.rows[slot, :len(t)].tolist() == t and (g.rows[slot, len(t):] == -1).all(), \
                    "the array of block-table rows has drifted from the tables"
