"""Reading and writing safetensors files by tensor name, in-tree.

Format (reference src/core/safetensors.cpp:16-44): 8 bytes little-endian
header length n, then n bytes of JSON `{name: {dtype, shape, data_offsets}}`
(the entry `__metadata__` is skipped), then the data; offsets are relative to
the end of the header. The reference re-opens the file for every tensor
(:48-56); here the file is mapped once and tensors are views of the mapping.
Beyond the reference's checks (header length :21-23, malformed entry :34-37)
the byte span of every entry is compared with its shape and dtype.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
import warnings
from dataclasses import dataclass
from typing import Dict, Iterable, Tuple

import torch


class WeightError(RuntimeError):
    """A checkpoint cannot be read or does not hold what the model needs."""


# safetensors dtype tag -> (torch dtype of the stored bytes, bytes per element)
_STORED = {
    "F32": (torch.float32, 4), "BF16": (torch.bfloat16, 2), "F16": (torch.float16, 2),
    "F64": (torch.float64, 8), "I64": (torch.int64, 8), "I32": (torch.int32, 4),
    "I16": (torch.int16, 2), "I8": (torch.int8, 1), "U8": (torch.uint8, 1),
    "BOOL": (torch.bool, 1),
}
_TAG_OF = {torch.float32: "F32", torch.bfloat16: "BF16", torch.float16: "F16",
           torch.float64: "F64", torch.int64: "I64", torch.int32: "I32"}


@dataclass(frozen=True)
class TensorInfo:
    dtype: str                 # safetensors tag as stored
    shape: Tuple[int, ...]
    begin: int                 # absolute byte offsets in the file
    end: int


def kept_dtype(tag: str) -> torch.dtype:
    """The dtype a stored tensor is kept in after loading: bfloat16 stays
    bfloat16, 32-bit floats stay 32-bit, float16/float64 become 32-bit floats
    (no precision is lost or invented silently), integer tables become int32."""
    if tag == "BF16":
        return torch.bfloat16
    if tag in ("F32", "F16", "F64"):
        return torch.float32
    if tag in ("I64", "I32", "I16", "I8", "U8"):
        return torch.int32
    raise WeightError(f"unsupported tensor dtype {tag}")


class SafeTensorsFile:
    """Index of one .safetensors file and zero-copy reads from its mapping."""

    def __init__(self, path: str):
        self.path = path
        if not os.path.isfile(path):
            raise WeightError(f"cannot open {path}: no such file")
        size = os.path.getsize(path)
        if size < 8:
            raise WeightError(f"{path}: too short for a safetensors header")
        self._file = open(path, "rb")
        (n,) = struct.unpack("<Q", self._file.read(8))
        if n == 0 or n > (1 << 30) or 8 + n > size:
            raise WeightError(f"{path}: bad safetensors header length {n}")
        try:
            header = json.loads(self._file.read(n).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise WeightError(f"{path}: safetensors header is not valid JSON ({e})") from None
        if not isinstance(header, dict):
            raise WeightError(f"{path}: safetensors header must be a JSON object")
        base = 8 + n
        self.tensors: Dict[str, TensorInfo] = {}
        for name, entry in header.items():
            if name == "__metadata__":
                continue
            try:
                tag = entry["dtype"]
                shape = tuple(int(x) for x in entry["shape"])
                b, e = (int(x) for x in entry["data_offsets"])
            except (KeyError, TypeError, ValueError):
                raise WeightError(f"{path}: malformed safetensors entry for '{name}'") from None
            if tag not in _STORED:
                raise WeightError(f"{path}: tensor '{name}' has unsupported dtype {tag}")
            count = 1
            for s in shape:
                count *= s
            if b < 0 or e < b or base + e > size or (e - b) != count * _STORED[tag][1]:
                raise WeightError(f"{path}: tensor '{name}' spans bytes [{b},{e}) but shape "
                                  f"{list(shape)} of {tag} needs {count * _STORED[tag][1]}")
            self.tensors[name] = TensorInfo(tag, shape, base + b, base + e)
        self._map = mmap.mmap(self._file.fileno(), 0, access=mmap.ACCESS_READ) if size else None

    def read(self, name: str) -> torch.Tensor:
        """The tensor as stored (a read-only view of the file mapping)."""
        info = self.tensors[name]
        dt, _ = _STORED[info.dtype]
        if info.end == info.begin:
            return torch.empty(info.shape, dtype=dt)
        buf = memoryview(self._map)[info.begin:info.end]
        with warnings.catch_warnings():
            warnings.simplefilter("ignore", UserWarning)  # the mapping is read-only on purpose
            return torch.frombuffer(buf, dtype=dt).reshape(info.shape)

    def close(self) -> None:
        if self._map is not None:
            try:
                self._map.close()
            except BufferError:
                pass  # views of the mapping are still alive; it goes with them
            self._map = None
        self._file.close()


def write_safetensors(path: str, tensors: Iterable[Tuple[str, torch.Tensor]]) -> None:
    """Write name -> tensor pairs as one .safetensors file (row-major, aligned
    header). Tensors are streamed: the iterable may generate them one by one."""
    items = []
    offset = 0
    tmp = path + ".data.tmp"
    with open(tmp, "wb") as data:
        for name, t in tensors:
            t = t.detach().to("cpu").contiguous()
            if t.dtype not in _TAG_OF:
                raise WeightError(f"cannot write tensor '{name}' of dtype {t.dtype}")
            raw = t.view(torch.uint8).numpy().tobytes() if t.numel() else b""
            items.append((name, {"dtype": _TAG_OF[t.dtype], "shape": list(t.shape),
                                 "data_offsets": [offset, offset + len(raw)]}))
            data.write(raw)
            offset += len(raw)
    header = json.dumps(dict(items), separators=(",", ":")).encode("utf-8")
    header += b" " * ((8 - len(header) % 8) % 8)
    with open(path, "wb") as out, open(tmp, "rb") as data:
        out.write(struct.pack("<Q", len(header)))
        out.write(header)
        while True:
            chunk = data.read(1 << 24)
            if not chunk:
                break
            out.write(chunk)
    os.remove(tmp)
