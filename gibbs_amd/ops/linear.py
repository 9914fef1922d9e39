"""y = x @ W^T for weights stored [out, in], in the precision of the run.

float32: the hand-written plain-FMA kernel (a true 32-bit product whose per-row result does not
depend on the batch).  bfloat16, float32 accumulation throughout: up to 64 rows take the
hand-written kernel that streams W once (decode); more rows take a matrix product on the matrix
cores, by default the library's (hipBLASLt, called directly; `GIBBS_GEMM=torch`: through
`torch.matmul`; the reference's engine uses a library product for its prefill as well), or the
hand-written tiled kernel (`GIBBS_GEMM=own`),
which also serves what the library does not give: float32 output (logits of many rows).
"""
from __future__ import annotations

import os
from typing import Optional

import torch

from . import PackedWeight, gemm_bf16, gemm_bf16_plain, gemm_f32, gemm_library, gemm_skinny, skinny_splits
from .lib import KernelError, require_cuda

# rows up to which the weight-streaming kernels are used (they re-read the activations once per 16
# output features, which stops paying beyond one or two MFMA tiles of rows)
SKINNY_ROWS = 32
# float32 logits: the few-row kernel streams the head matrix faster than the tiled product up to here
SKINNY_ROWS_F32_OUT = 48
USE_LIBRARY_GEMM = os.environ.get("GIBBS_GEMM", "library") != "own"
# the library product is hipBLASLt called directly (its heuristic's choice kept per shape: a call costs
# the host 12 us instead of the 20 us of torch.matmul); "torch" goes through PyTorch
LIBRARY_THROUGH_TORCH = os.environ.get("GIBBS_GEMM", "library") == "torch"


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
    if x.dtype == torch.float32:
        if out_dtype != torch.float32:
            raise KernelError("linear: the float32 path writes float32")
        return gemm_f32(x, w)
    if x.dtype == torch.bfloat16:
        n, i = x.shape
        if i % 8 or w.stride(0) % 8 or (n > 1 and x.stride(0) % 8) or x.data_ptr() % 16 or w.data_ptr() % 16:
            return gemm_bf16_plain(x, w, out_dtype)             # what the matrix-core kernels refuse
        if 1 <= x.shape[0] <= (SKINNY_ROWS_F32_OUT if out_dtype == torch.float32 and not partial_ok else SKINNY_ROWS):
            splits = skinny_splits(w.shape[0], w.shape[1]) if partial_ok else 1
            return gemm_skinny(x, w if packed is None else packed, out_dtype, splits)
        if USE_LIBRARY_GEMM and out_dtype == torch.bfloat16:
            return torch.matmul(x, w.t()) if LIBRARY_THROUGH_TORCH else gemm_library(x, w)
        return gemm_bf16(x, w, out_dtype)
    raise KernelError(f"linear: unsupported dtype {x.dtype}")
