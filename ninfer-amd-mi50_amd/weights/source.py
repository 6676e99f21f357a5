"""Where a model's tensors come from: a checkpoint folder or a seeded
generator. Both answer `shapes()` and `read(name)`; the model asks by name.

Checkpoint folders (reference src/models/model.hip:85-113): the unique files
of `model.safetensors.index.json`'s `weight_map` if that file exists, else
`model.safetensors`; every file's header is indexed into name -> file.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

import torch

from .safetensors_io import SafeTensorsFile, WeightError, kept_dtype


@dataclass(frozen=True)
class TensorSpec:
    """What a part expects of one checkpoint tensor.

    role: 'matrix' (kept in the compute dtype), 'gain' (norm weight, read in
    32-bit, random values 1 + N(0, s)), 'bias' (read in 32-bit).
    """
    shape: Tuple[int, ...]
    role: str = "matrix"


class CheckpointSource:
    """Tensors of a model folder, read by name."""

    def __init__(self, model_dir: str):
        self.model_dir = model_dir
        index_path = os.path.join(model_dir, "model.safetensors.index.json")
        if os.path.isfile(index_path):
            with open(index_path, "r", encoding="utf-8") as f:
                try:
                    weight_map = json.load(f)["weight_map"]
                except (json.JSONDecodeError, KeyError, TypeError):
                    raise WeightError(f"{index_path}: no usable 'weight_map'") from None
            names = sorted(set(weight_map.values()))
        else:
            names = ["model.safetensors"]
        self.files: List[SafeTensorsFile] = []
        self._where: Dict[str, SafeTensorsFile] = {}
        for fn in names:
            f = SafeTensorsFile(os.path.join(model_dir, fn))
            self.files.append(f)
            for name in f.tensors:
                self._where[name] = f

    def shapes(self) -> Dict[str, Tuple[int, ...]]:
        return {n: f.tensors[n].shape for n, f in self._where.items()}

    def read(self, name: str) -> torch.Tensor:
        """CPU tensor in its kept dtype (bfloat16 stays, 32-bit stays, integer
        tables become int32)."""
        if name not in self._where:
            raise WeightError(f"missing tensor in checkpoint: {name}")
        f = self._where[name]
        t = f.read(name)
        want = kept_dtype(f.tensors[name].dtype)
        return t if t.dtype == want else t.to(want)

    def close(self) -> None:
        for f in self.files:
            f.close()


class RandomSource:
    """Seeded random tensors for a set of expected tensors.

    Every element is a pure function of (seed, tensor name, flat index): a
    counter hash turned into an approximately normal number (the sum of twelve
    uniform ones, see counter_random.py). Matrices and biases: std * z; gains:
    1 + std * z. A tensor's values do not depend on which other tensors exist,
    on the order they are asked for, or on where they are made: on 'cpu' the
    host computes them, on a GPU device the library's fill kernel does, and
    both give the same bits. That is how models too large to write to disk are
    filled, and how a test can know what such a model holds.
    """

    def __init__(self, specs: Dict[str, TensorSpec], seed: int, dtype: torch.dtype,
                 std: float = 0.02, device: str = "cpu", ops=None):
        self.specs = specs
        self.seed = int(seed)
        self.dtype = dtype
        self.std = std
        self.device = device
        self._ops = ops

    def shapes(self) -> Dict[str, Tuple[int, ...]]:
        return {n: s.shape for n, s in self.specs.items()}

    def read(self, name: str) -> torch.Tensor:
        from . import counter_random
        if name not in self.specs:
            raise WeightError(f"missing tensor in checkpoint: {name}")
        spec = self.specs[name]
        key = counter_random.tensor_key(self.seed, name)
        mean = 1.0 if spec.role == "gain" else 0.0
        if torch.device(self.device).type == "cpu":
            return counter_random.fill(spec.shape, key, self.std, mean).to(self.dtype)
        if self._ops is None:
            from ..kernels import load_ops
            self._ops = load_ops()
        t = torch.empty(spec.shape, dtype=self.dtype, device=self.device)
        self._ops.fill_random(t, key, self.std, mean)
        return t

    def close(self) -> None:
        pass


def check_tensors(have: Dict[str, Tuple[int, ...]], want: Dict[str, TensorSpec],
                  where: str, unused: Optional[Dict[str, TensorSpec]] = None) -> None:
    """One error that lists every missing tensor, every unexpected tensor and
    every tensor of the wrong shape (the reference stops at the first missing
    name, src/models/model.hip:115-119, and checks no shapes). Names in
    `unused` may be there or not; if there, their shape is checked too."""
    known = dict(unused or {})
    known.update(want)
    missing = sorted(n for n in want if n not in have)
    unexpected = sorted(n for n in have if n not in known)
    wrong = sorted((n, tuple(have[n]), tuple(known[n].shape)) for n in known
                   if n in have and tuple(have[n]) != tuple(known[n].shape))
    if not (missing or unexpected or wrong):
        return
    lines = [f"{where}: checkpoint does not match the model"]
    if missing:
        lines.append(f"  missing tensors ({len(missing)}):")
        lines += [f"    {n}  expected shape {list(want[n].shape)}" for n in missing]
    if unexpected:
        lines.append(f"  unexpected tensors ({len(unexpected)}):")
        lines += [f"    {n}  shape {list(have[n])}" for n in unexpected]
    if wrong:
        lines.append(f"  wrong shapes ({len(wrong)}):")
        lines += [f"    {n}  has {list(h)}, expected {list(w)}" for n, h, w in wrong]
    raise WeightError("\n".join(lines))
