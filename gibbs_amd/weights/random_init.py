"""Random-weights mode: a model folder (config.json, model.safetensors) from a
configuration and a seed.

Every tensor has its own stream seeded by hash(name) ^ seed, so values do not depend on the
order tensors are written in: the idea of the reference's synthetic checkpoints
(src/arch/load.rs:2355-2420, per-name seed :1410), with a normal
distribution of standard deviation 0.02 instead of its uniform +-0.02.
"""
from __future__ import annotations

import hashlib
import json
import os
from typing import Dict, Iterable

import torch

from ..config.base import ArchConfig
from .loader import COMPUTE, FLOAT32, INT32, TensorDecl
from .safetensors_io import write_safetensors


def _stream(name: str, seed: int) -> torch.Generator:
    h = int.from_bytes(hashlib.sha256(name.encode()).digest()[:8], "little")
    g = torch.Generator(device="cpu")
    g.manual_seed((h ^ (seed * 0x9E3779B97F4A7C15)) & ((1 << 63) - 1))
    return g


def random_tensor(decl: TensorDecl, seed: int, store_dtype: torch.dtype, std: float = 0.02,
                  gain_std: float = 0.0, bias_std: float = 0.02) -> torch.Tensor:
    g = _stream(decl.name, seed)
    if decl.dtype == INT32:
        return torch.zeros(decl.shape, dtype=torch.int32)
    if decl.init == "gain":
        t = torch.ones(decl.shape, dtype=torch.float32)
        if gain_std > 0:
            t += torch.randn(decl.shape, generator=g, dtype=torch.float32) * gain_std
    elif decl.init == "bias":
        t = torch.randn(decl.shape, generator=g, dtype=torch.float32) * bias_std
    elif decl.init == "zeros":
        t = torch.zeros(decl.shape, dtype=torch.float32)
    else:
        t = torch.randn(decl.shape, generator=g, dtype=torch.float32) * std
    keep32 = decl.dtype == FLOAT32 or len(decl.shape) <= 1
    return t if keep32 else t.to(store_dtype)


def write_random_model(folder: str, config: ArchConfig, decls: Iterable[TensorDecl], seed: int,
                       dtype: str = "bfloat16", std: float = 0.02, gain_std: float = 0.0,
                       bias_std: float = 0.02) -> None:
    """Matrices are stored in `dtype`, gains and biases in float32."""
    store = {"bfloat16": torch.bfloat16, "float32": torch.float32, "float16": torch.float16}[dtype]
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(config.to_dict(), f, indent=1)
    tensors = ((d.name, random_tensor(d, seed, store, std, gain_std, bias_std)) for d in decls)
    write_safetensors(os.path.join(folder, "model.safetensors"), list(tensors))


def random_weights_on_device(decls: Iterable[TensorDecl], seed: int, compute_dtype: torch.dtype,
                             device: torch.device | str, std: float = 0.02, gain_std: float = 0.0,
                             bias_std: float = 0.02):
    """The same kinds of random tensors, made on the device without a model folder (benchmarks of
    large shapes).  Values differ from the folder mode's: the device has its own generator."""
    from .loader import WeightStore
    device = torch.device(device)
    out: Dict[str, torch.Tensor] = {}
    for d in decls:
        g = torch.Generator(device=device)
        g.manual_seed(_stream(d.name, seed).initial_seed())
        want = d.resolved_dtype(compute_dtype)
        if d.dtype == INT32:
            out[d.name] = torch.zeros(d.shape, dtype=torch.int32, device=device)
        elif d.init == "gain":
            t = torch.ones(d.shape, dtype=torch.float32, device=device)
            if gain_std > 0:
                t += torch.randn(d.shape, generator=g, dtype=torch.float32, device=device) * gain_std
            out[d.name] = t.to(want)
        elif d.init == "zeros":
            out[d.name] = torch.zeros(d.shape, dtype=want, device=device)
        else:
            scale = bias_std if d.init == "bias" else std
            out[d.name] = (torch.randn(d.shape, generator=g, dtype=torch.float32, device=device) * scale).to(want)
    return WeightStore(out, compute_dtype, device)
