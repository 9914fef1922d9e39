"""Weights by tensor name, checked against what the model declares.

Every part of a model declares the tensors it reads (`TensorDecl`).  Loading compares the
declarations with the checkpoint's table and fails once, listing every missing tensor,
every tensor nobody reads, and every wrong shape: the reference refuses unread checkpoint
tensors (src/runtime/lm.rs:357-367) and missing ones
(src/arch/build.rs:454-457) separately.

Precision policy: floating matrices are kept in the compute dtype of the run (bfloat16, or
float32 for the true 32-bit path); tensors of rank <= 1 (gains, biases) are float32, as in
the reference (src/arch/load.rs:902-917); a declaration can pin float32 for
a tensor whatever its rank; integer tables become int32.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Iterable, List, Optional, Sequence, Tuple

import torch

from .safetensors_io import open_checkpoint

COMPUTE = "compute"
FLOAT32 = "float32"
INT32 = "int32"


@dataclass(frozen=True)
class TensorDecl:
    name: str
    shape: Tuple[int, ...]
    dtype: str = COMPUTE                    # COMPUTE | FLOAT32 | INT32
    init: str = "normal"                    # random-weights mode: normal | gain | bias | zeros
    alt_shapes: Tuple[Tuple[int, ...], ...] = ()   # other stored shapes of the same data

    def resolved_dtype(self, compute_dtype: torch.dtype) -> torch.dtype:
        if self.dtype == INT32:
            return torch.int32
        if self.dtype == FLOAT32 or len(self.shape) <= 1:
            return torch.float32
        return compute_dtype


class WeightError(ValueError):
    """The checkpoint does not fit the model; lists everything that is wrong."""

    def __init__(self, missing: Sequence[str], unexpected: Sequence[str],
                 wrong_shape: Sequence[Tuple[str, Tuple[int, ...], Tuple[int, ...]]], where: str = ""):
        self.missing, self.unexpected, self.wrong_shape = list(missing), list(unexpected), list(wrong_shape)
        lines = [f"checkpoint {where} does not fit the model:".replace("  ", " ")]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  checkpoint tensors no part reads ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong_shape:
            lines.append(f"  wrong shapes ({len(self.wrong_shape)}): " + ", ".join(
                f"{n} is {list(got)}, expected {list(want)}" for n, got, want in self.wrong_shape))
        super().__init__("\n".join(lines))


def check_table(decls: Iterable[TensorDecl], table: Dict[str, Tuple[int, ...]], where: str = "") -> None:
    """Raises one WeightError that lists all differences between declarations and table."""
    decls = list(decls)
    seen = set()
    dup = [d.name for d in decls if d.name in seen or seen.add(d.name)]
    if dup:
        raise ValueError(f"tensors declared twice by the model: {dup}")
    missing = [d.name for d in decls if d.name not in table]
    unexpected = sorted(set(table) - {d.name for d in decls})
    wrong = [(d.name, tuple(table[d.name]), d.shape) for d in decls
             if d.name in table and tuple(table[d.name]) != d.shape and tuple(table[d.name]) not in d.alt_shapes]
    if missing or unexpected or wrong:
        raise WeightError(missing, unexpected, wrong, where)


class WeightStore:
    """Tensors on the device, by name, in the dtype their declaration resolves to."""

    def __init__(self, tensors: Dict[str, torch.Tensor], compute_dtype: torch.dtype, device: torch.device):
        self._t = tensors
        self.compute_dtype = compute_dtype
        self.device = device

    def __getitem__(self, name: str) -> torch.Tensor:
        return self._t[name]

    def __contains__(self, name: str) -> bool:
        return name in self._t

    def names(self) -> List[str]:
        return list(self._t)

    def nbytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self._t.values())


def load_weights(model_dir: str, decls: Iterable[TensorDecl], compute_dtype: torch.dtype,
                 device: torch.device | str) -> WeightStore:
    """Reads exactly the declared tensors, one at a time, onto `device`."""
    decls = list(decls)
    table, files = open_checkpoint(model_dir)
    check_table(decls, {n: e.shape for n, e in table.items()}, where=model_dir)
    device = torch.device(device)
    out: Dict[str, torch.Tensor] = {}
    for d in decls:
        e = table[d.name]
        t = files[e.file].read(d.name)
        want = d.resolved_dtype(compute_dtype)
        if want == torch.int32 and t.dtype.is_floating_point:
            raise WeightError([], [], [], where=f"{model_dir}: {d.name} is stored as {e.dtype}, an integer table was expected")
        t = t.reshape(d.shape)
        out[d.name] = t.to(device=device, dtype=want).contiguous()
    return WeightStore(out, compute_dtype, device)


def table_of(model_dir: str) -> Dict[str, Tuple[int, ...]]:
    """name -> shape of a model folder's checkpoint, without reading data."""
    table, _ = open_checkpoint(model_dir)
    return {n: e.shape for n, e in table.items()}
