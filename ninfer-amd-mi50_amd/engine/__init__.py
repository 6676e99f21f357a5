from .runner import Chunk, ModelRunner

__all__ = ["Chunk", "ModelRunner"]
