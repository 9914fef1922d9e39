"""y = x @ W^T for weights stored [out, in], in the precision of the run.

float32: the hand-written plain-FMA kernel (a true 32-bit product whose per-row result does not
depend on the batch).  bfloat16: float32 accumulation; the output is bfloat16, or float32 where
the caller asks for it (logits).
"""
from __future__ import annotations

from typing import Optional

import torch

from . import gemm_bf16, gemm_f32
from .lib import KernelError, require_cuda


def linear(x: torch.Tensor, w: torch.Tensor, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    require_cuda(x, w)
    if x.dtype != w.dtype:
        raise KernelError(f"linear: activations are {x.dtype}, weights {w.dtype}")
    out_dtype = out_dtype or x.dtype
    if x.dtype == torch.float32:
        if out_dtype != torch.float32:
            raise KernelError("linear: the float32 path writes float32")
        return gemm_f32(x, w)
    if x.dtype == torch.bfloat16:
        return gemm_bf16(x, w, out_dtype)
    raise KernelError(f"linear: unsupported dtype {x.dtype}")
