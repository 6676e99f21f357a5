"""ninfer for MI355X: a small, whole inference engine for Qwen2-MoE on one
gfx950 GPU: typed configuration and a model registry, weights from
safetensors, models put together from parts, a paged cache, one step
function, a scheduler with sampling, and hand-written HIP kernels."""
from . import models  # noqa: F401  (registers the architectures)
from .config import ConfigError, EngineOptions, Qwen2MoeConfig
from .api import Ninfer, Session
from .engine import Chunk, ModelRunner
from .engine.scheduler import Request, Scheduler
from .sampling import Sampler, SamplingParams
from .loading import build_spec, load_model, random_model, write_random_model
from .registry import (architectures, make_part, register_architecture, register_part,
                       resolve_architecture)
from .weights import WeightError

__all__ = ["Ninfer", "Session", "Request", "Scheduler", "Sampler", "SamplingParams", "ConfigError", "EngineOptions", "Qwen2MoeConfig", "Chunk", "ModelRunner", "build_spec",
           "load_model", "random_model", "write_random_model", "architectures", "make_part",
           "register_architecture", "register_part", "resolve_architecture", "WeightError"]
