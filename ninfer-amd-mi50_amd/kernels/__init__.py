"""Loading of the hand-written gfx950 kernel library. There is no fallback:
without a GPU or without the library the engine does not run."""
from __future__ import annotations

from .build import build, ensure_built
from .ops import HipOps, KernelError

_OPS = None


def load_ops() -> HipOps:
    """The kernel library, built on first use if no built library matches the
    sources. Raises if there is no GPU or the library cannot be built or loaded."""
    global _OPS
    if _OPS is None:
        import torch
        if not torch.cuda.is_available():
            raise RuntimeError("ninfer needs a GPU: the engine has no CPU path "
                               "(torch.cuda.is_available() is False)")
        _OPS = HipOps(ensure_built())
    return _OPS


__all__ = ["build", "ensure_built", "load_ops", "HipOps", "KernelError"]
