"""y = x @ W^T for weights stored [out, in], in the precision of the run.

Which kernel runs is decided in one place, the native step (csrc/step_plan.hip, `choose_linear`), and
this function asks there: float32 takes the hand-written plain-FMA kernel (a true 32-bit product whose
per-row result does not depend on the batch); bfloat16, with float32 accumulation throughout, takes the
hand-written kernel that streams W once for few rows (decode), and for more rows a matrix product on the
matrix cores, by default the library's (hipBLASLt, called directly; the reference's engine uses a
library product for its prefill as well), or the hand-written tiled kernel (`GIBBS_GEMM=own`), which
also serves what the library does not give: float32 output (logits of many rows).
"""
from __future__ import annotations

import os
from typing import Optional

import torch

from . import PackedWeight
from .lib import KernelError, call, dtype_code, library, ptr, require_cuda, stream

USE_LIBRARY_GEMM = os.environ.get("GIBBS_GEMM", "library") != "own"


def linear(x: torch.Tensor, w: torch.Tensor, out_dtype: Optional[torch.dtype] = None,
           partial_ok: bool = False, packed: Optional[PackedWeight] = None) -> torch.Tensor:
    """`partial_ok`: the caller can take float32 partial sums [S, N, O] (to be added in order)
    instead of the finished product; the few-row kernel then also splits k over workgroups when
    the output alone is too narrow to fill the chip.  `packed`: the same matrix in the order the
    few-row kernel reads fastest, used when that kernel is the one that runs."""
    require_cuda(x, w)
    if x.dtype != w.dtype:
        raise KernelError(f"linear: activations are {x.dtype}, weights {w.dtype}")
    out_dtype = out_dtype or x.dtype
    if x.dtype == torch.float32 and out_dtype != torch.float32:
        raise KernelError("linear: the float32 path writes float32")
    if x.dtype not in (torch.float32, torch.bfloat16) or out_dtype not in (x.dtype, torch.float32):
        raise KernelError(f"linear: unsupported dtypes {x.dtype} -> {out_dtype}")
    assert x.dim() == 2 and w.dim() == 2 and x.shape[1] == w.shape[1] and x.stride(1) == 1 and w.is_contiguous(), (x.shape, w.shape)
    if packed is not None and packed.groups != 1:
        raise KernelError("linear: the weights are packed in row groups")
    n, i = x.shape
    o = w.shape[0]
    ldx = x.stride(0) if n > 1 else i
    f32_out, own = int(out_dtype == torch.float32), int(not USE_LIBRARY_GEMM)
    splits = library().gibbs_linear_splits(dtype_code(x.dtype), n, o, i, ldx, ptr(x), ptr(w), f32_out, int(partial_ok), own)
    out = torch.empty((splits, n, o) if splits > 1 else (n, o), dtype=torch.float32 if splits > 1 else out_dtype, device=x.device)
    call("gibbs_linear", ptr(x), ldx, ptr(w), None if packed is None else packed.data_ptr(), ptr(out), dtype_code(x.dtype), n, o, i,
         f32_out, int(partial_ok), own, stream())
    return out
