"""Runtime options of an engine, as distinct from the model's configuration.

Successor of the reference's `ModelOptions` (src/models/model.h:37-50:
max_context 32768, prefill_chunk 512, num_sequences 1, use_graph false) with
what a paged cache and a true 32-bit path add.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional


@dataclass
class EngineOptions:
    dtype: str = "bfloat16"        # "bfloat16" or "float32": storage of weights, activations, cache
    max_context: int = 32768       # most tokens one request may hold (reference --max-context)
    prefill_chunk: int = 512       # token budget of one step (reference --prefill-chunk)
    num_sequences: int = 8         # most live requests (reference num_sequences)
    page_size: int = 16            # tokens per cache page
    num_pages: Optional[int] = None  # pages per cache group; None: from kv_bytes, else enough for every request at max_context
    kv_bytes: Optional[int] = None   # bytes of paged cache over all layers (the reference sizes its slabs in bytes, src/api/ninfer_c_api.cpp:105-108)
    use_graph: bool = False        # replay decode-only steps from a captured HIP graph
    max_graphs: int = 32           # most captured graphs kept (one per count of requests and context bound); the least recently replayed goes first
    poison_freed_pages: bool = False  # debugging: fill pages that are given back with NaN
    check_pages: bool = False      # debugging: before every step, check on the host that every page the step reads or writes is held by its request and by no other
    device: str = "cuda:0"

    def validate(self) -> None:
        if self.dtype not in ("bfloat16", "float32"):
            raise ValueError(f"dtype must be 'bfloat16' or 'float32', got {self.dtype!r}")
        for name in ("max_context", "prefill_chunk", "num_sequences", "page_size", "max_graphs"):
            if getattr(self, name) < 1:
                raise ValueError(f"{name} must be >= 1, got {getattr(self, name)}")
        if self.num_pages is not None and self.num_pages < 1:
            raise ValueError(f"num_pages must be >= 1, got {self.num_pages}")
        if self.kv_bytes is not None and self.kv_bytes < 1:
            raise ValueError(f"kv_bytes must be >= 1, got {self.kv_bytes}")
        if self.kv_bytes is not None and self.num_pages is not None:
            raise ValueError("give num_pages or kv_bytes, not both")
        self.warn_of_slow_pages(self.page_size)

    def warn_of_slow_pages(self, page_size: int) -> None:
        """Warns of a page size (the engine's, or one a mixer asks for) with which bfloat16
        attention runs the plain kernel."""
        if self.dtype == "bfloat16" and not self.page_size_suits_fast_attention(page_size):
            import warnings
            warnings.warn(
                f"page_size {page_size}: the matrix-core attention kernels take pages of "
                f"8, 16, 32 or 64 tokens (4 too with heads of 128); with this size every bfloat16 step runs the plain "
                f"attention kernel (one wave per row and head), which is right and many times "
                f"slower", stacklevel=3)

    def page_size_suits_fast_attention(self, page_size: Optional[int] = None) -> bool:
        """The bfloat16 prompt kernel walks keys in tiles of 64 that whole pages must fill, one of
        its loads (1 KB of a head's rows: 4 rows of heads of 128, 8 of 64) must stay inside a
        page, and both fast kernels find a key's page by a shift: a power of two from 4 to 64
        (pages of 4 with heads of 64 still run the plain kernel for prompt portions)."""
        ps = self.page_size if page_size is None else page_size
        return ps >= 4 and ps & (ps - 1) == 0 and ps <= 64

    def pages_per_request(self) -> int:
        return -(-self.max_context // self.page_size)

    def pool_pages(self, bytes_per_token: int = 0) -> int:
        """Pages of every cache group. `bytes_per_token`: what one token takes in the paged
        cache over all layers (needed only with kv_bytes)."""
        if self.num_pages is not None:
            return self.num_pages
        if self.kv_bytes is not None:
            pages = self.kv_bytes // max(1, bytes_per_token * self.page_size)
            if pages < 1:
                raise ValueError(f"kv_bytes {self.kv_bytes} holds no page of {self.page_size} "
                                 f"tokens ({bytes_per_token} bytes a token)")
            return int(pages)
        return self.pages_per_request() * self.num_sequences
