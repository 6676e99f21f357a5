"""From a model folder (or a configuration and a seed) to a bound model.

`load_model` reads config.json, resolves `architectures[0]` in the registry,
builds the model from its typed configuration, checks the checkpoint's tensor
names and shapes against what the model's parts expect, and binds the
weights. The reference's counterpart is `Model::Impl::load`
(src/models/model.hip:833-948).
"""
from __future__ import annotations

import json
import os
from typing import Any, Dict, Optional

import torch

from . import models  # noqa: F401  (registers the architectures)
from .config.base import architecture_name, read_config_json
from .config.options import EngineOptions
from .engine.runner import ModelRunner
from .registry import resolve_architecture
from .weights.safetensors_io import write_safetensors
from .weights.source import CheckpointSource, RandomSource

_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32}


def build_spec(raw_config: Dict[str, Any]):
    """(typed configuration, ModelSpec) for a raw config.json dictionary."""
    read_config, build = resolve_architecture(architecture_name(raw_config))
    cfg = read_config(raw_config)
    return cfg, build(cfg)


def load_model(model_dir: str, options: Optional[EngineOptions] = None, ops=None) -> ModelRunner:
    """A runner (bound model + cache + step function) for a model folder."""
    options = options or EngineOptions()
    raw = read_config_json(model_dir)
    cfg, spec = build_spec(raw)
    source = CheckpointSource(model_dir)
    try:
        runner = ModelRunner(spec, source, options, ops=ops, where=model_dir)
    finally:
        source.close()
    runner.config = cfg
    return runner


def random_model(raw_config: Dict[str, Any], seed: int, options: Optional[EngineOptions] = None,
                 ops=None, weights_dtype: Optional[str] = None, std: float = 0.02) -> ModelRunner:
    """A runner with seeded random weights generated on the engine's device
    (for models too large to write to disk). `weights_dtype`: the precision the values are
    rounded to before the engine takes them (default: the engine's own), so that a 32-bit
    engine can hold exactly the weights of a bfloat16 one. The values are those that
    `write_random_model` would store for the same configuration, seed and std, bit for bit;
    `runner.tensor(name)` reads them back."""
    options = options or EngineOptions()
    cfg, spec = build_spec(raw_config)
    source = RandomSource(spec.tensor_specs(), seed, _DTYPES[weights_dtype or options.dtype],
                          std=std, device=options.device, ops=ops)
    runner = ModelRunner(spec, source, options, ops=ops, where="random weights")
    runner.config = cfg
    return runner


def write_random_model(model_dir: str, raw_config: Dict[str, Any], seed: int,
                       dtype: str = "float32", std: float = 0.02) -> None:
    """Random-weights mode: write config.json and model.safetensors for a
    configuration and a seed (values N(0, std); norm gains 1 + N(0, std))."""
    if dtype not in _DTYPES:
        raise ValueError(f"dtype must be one of {sorted(_DTYPES)}, got {dtype!r}")
    _, spec = build_spec(raw_config)
    source = RandomSource(spec.tensor_specs(), seed, _DTYPES[dtype], std=std, device="cpu")
    os.makedirs(model_dir, exist_ok=True)
    with open(os.path.join(model_dir, "config.json"), "w", encoding="utf-8") as f:
        json.dump(raw_config, f, indent=1)
    write_safetensors(os.path.join(model_dir, "model.safetensors"),
                      ((name, source.read(name)) for name in sorted(source.specs)))
