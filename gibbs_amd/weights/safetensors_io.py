"""Reading and writing safetensors files without touching tensor data until it is asked for.

Layout (src/model/loaders/safetensors.rs:15-64): an unsigned 64-bit
little-endian header length, a JSON header {name: {dtype, shape, data_offsets}}, then the
data.  Sharded checkpoints name their files in `model.safetensors.index.json`
(src/arch/load.rs:365).
"""
from __future__ import annotations

import json
import mmap
import os
from dataclasses import dataclass
from typing import Dict, Iterable, Mapping, Tuple

import numpy as np
import torch

_TORCH_DTYPES = {
    "F32": torch.float32, "BF16": torch.bfloat16, "F16": torch.float16, "F64": torch.float64,
    "I32": torch.int32, "I64": torch.int64, "I16": torch.int16, "I8": torch.int8, "U8": torch.uint8,
    "BOOL": torch.bool,
}
_TAGS = {v: k for k, v in _TORCH_DTYPES.items()}


@dataclass(frozen=True)
class TensorEntry:
    name: str
    dtype: str                      # safetensors tag, e.g. "BF16"
    shape: Tuple[int, ...]
    file: str
    begin: int                      # byte offsets inside the file
    end: int


class SafetensorsFile:
    """One file: its table, and tensors read one at a time from a memory map."""

    def __init__(self, path: str):
        self.path = path
        with open(path, "rb") as f:
            head = f.read(8)
            if len(head) < 8:
                raise ValueError(f"{path}: not a safetensors file (shorter than 8 bytes)")
            n = int.from_bytes(head, "little")
            size = os.path.getsize(path)
            if n <= 0 or 8 + n > size:
                raise ValueError(f"{path}: header length {n} does not fit the file ({size} bytes)")
            header = json.loads(f.read(n))
        self.entries: Dict[str, TensorEntry] = {}
        base = 8 + n
        for name, meta in header.items():
            if name == "__metadata__":
                continue
            lo, hi = meta["data_offsets"]
            if meta["dtype"] not in _TORCH_DTYPES:
                raise ValueError(f"{path}: tensor {name} has unsupported dtype {meta['dtype']}")
            self.entries[name] = TensorEntry(name, meta["dtype"], tuple(int(s) for s in meta["shape"]),
                                             path, base + lo, base + hi)
        self._map = None

    def read(self, name: str) -> torch.Tensor:
        """A CPU tensor that owns its memory (a copy out of the map)."""
        e = self.entries[name]
        if self._map is None:
            with open(self.path, "rb") as f:
                self._map = mmap.mmap(f.fileno(), 0, access=mmap.ACCESS_COPY)
        dtype = _TORCH_DTYPES[e.dtype]
        count = int(np.prod(e.shape)) if e.shape else 1
        if count == 0:
            return torch.empty(e.shape, dtype=dtype)
        flat = torch.frombuffer(memoryview(self._map)[e.begin:e.end], dtype=dtype, count=count)
        return flat.reshape(e.shape).clone()


def open_checkpoint(model_dir: str) -> Tuple[Dict[str, TensorEntry], Dict[str, SafetensorsFile]]:
    """The tensor table of a model folder (single file or index of shards) and its files."""
    single = os.path.join(model_dir, "model.safetensors")
    index = os.path.join(model_dir, "model.safetensors.index.json")
    files: Dict[str, SafetensorsFile] = {}
    table: Dict[str, TensorEntry] = {}
    if os.path.isfile(single):
        names = [single]
    elif os.path.isfile(index):
        with open(index) as f:
            shard_of = json.load(f)["weight_map"]
        names = sorted({os.path.join(model_dir, s) for s in shard_of.values()})
    else:
        raise FileNotFoundError(f"{model_dir}: no model.safetensors or model.safetensors.index.json")
    for path in names:
        sf = SafetensorsFile(path)
        files[path] = sf
        for name, entry in sf.entries.items():
            if name in table:
                raise ValueError(f"tensor {name} appears in {table[name].file} and in {path}")
            table[name] = entry
    return table, files


def write_safetensors(path: str, tensors: Mapping[str, torch.Tensor] | Iterable[Tuple[str, torch.Tensor]]) -> None:
    """Writes CPU tensors in the order given; the header is padded to 8 bytes with spaces."""
    items = list(tensors.items()) if isinstance(tensors, Mapping) else list(tensors)
    header, offset = {}, 0
    for name, t in items:
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _TAGS[t.dtype], "shape": list(t.shape), "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
    blob = json.dumps(header, separators=(",", ":")).encode()
    blob += b" " * ((8 - len(blob) % 8) % 8)
    with open(path, "wb") as f:
        f.write(len(blob).to_bytes(8, "little"))
        f.write(blob)
        for _, t in items:
            t = t.detach().contiguous().cpu()
            f.write(t.view(torch.uint8).numpy().tobytes() if t.numel() else b"")
