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
    num_pages: Optional[int] = None  # pages per cache group; None: enough for every request at max_context
    use_graph: bool = False        # replay decode-only steps from a captured HIP graph
    poison_freed_pages: bool = False  # debugging: fill pages that are given back with NaN
    device: str = "cuda:0"

    def validate(self) -> None:
        if self.dtype not in ("bfloat16", "float32"):
            raise ValueError(f"dtype must be 'bfloat16' or 'float32', got {self.dtype!r}")
        for name in ("max_context", "prefill_chunk", "num_sequences", "page_size"):
            if getattr(self, name) < 1:
                raise ValueError(f"{name} must be >= 1, got {getattr(self, name)}")
        if self.num_pages is not None and self.num_pages < 1:
            raise ValueError(f"num_pages must be >= 1, got {self.num_pages}")

    def pages_per_request(self) -> int:
        return -(-self.max_context // self.page_size)

    def pool_pages(self) -> int:
        if self.num_pages is not None:
            return self.num_pages
        return self.pages_per_request() * self.num_sequences
