"""Loads the HIP kernel library and declares its C interface.

There is no fallback: if the library cannot be found or built, or a kernel call reports an
error, an exception says so.
"""
from __future__ import annotations

import ctypes
import threading
from ctypes import c_float, c_int, c_long, c_void_p

from typing import Optional

import torch

from .. import build as _build

ABI_VERSION = 1
_lock = threading.Lock()
_lib = None


class KernelError(RuntimeError):
    """A kernel entry point refused its arguments or its launch failed."""


_SIGNATURES = {
    "gibbs_embed": [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p],
    "gibbs_add_rmsnorm": [c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_int, c_void_p, c_int, c_int, c_void_p],
    "gibbs_residual_add": [c_void_p, c_void_p, c_int, c_int, c_long, c_void_p, c_long, c_void_p],
    "gibbs_gemm_f32": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_long, c_long, c_long, c_void_p],
    "gibbs_gemm_bf16_plain": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_long, c_long, c_long, c_void_p],
    "gibbs_gemm_bf16": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_long, c_long, c_long, c_void_p],
    "gibbs_gemm_skinny": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_long, c_long, c_long, c_int,
                          c_void_p],
    "gibbs_add_partials_rmsnorm": [c_void_p, c_void_p, c_int, c_long, c_void_p, c_float, c_void_p, c_int, c_void_p,
                                   c_int, c_int, c_void_p],
    "gibbs_skinny_store": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_long, c_long, c_long, c_int, c_float,
                           c_void_p],
    "gibbs_skinny_residual": [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_long, c_long, c_void_p],
    "gibbs_skinny_glu": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_long, c_long, c_long, c_int, c_float,
                         c_int, c_void_p],
    "gibbs_skinny_conv": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_long, c_long, c_int, c_float, c_void_p,
                          c_void_p, c_void_p, c_long, c_void_p, c_void_p, c_int, c_void_p],
    "gibbs_attention_decode_fused": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                     c_float, c_void_p, c_int, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                                     c_int, c_int, c_int, c_int, c_long, c_long, c_float, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "gibbs_glu": [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p],
    "gibbs_shortconv": [c_void_p, c_void_p, c_void_p, c_void_p, c_long, c_void_p, c_void_p, c_void_p, c_void_p,
                        c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "gibbs_rope_table": [c_void_p, c_void_p, c_int, c_int, c_void_p],
    "gibbs_qk_rope_kv": [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_float, c_void_p, c_int, c_int,
                         c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_long,
                         c_void_p],
    "gibbs_attention_plain": [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int,
                              c_int, c_int, c_int, c_int, c_int, c_int, c_long, c_long, c_float, c_int, c_void_p, c_void_p],
    "gibbs_decode_tail": [c_void_p, c_int, c_long, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p,
                          c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p],
    "gibbs_attention_decode": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                               c_int, c_int, c_int, c_int, c_int, c_int, c_long, c_long, c_float, c_int, c_int,
                               c_int, c_int, c_int, c_void_p],
    "gibbs_attention_prefill": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                                c_int, c_int, c_int, c_int, c_int, c_long, c_long, c_float, c_int, c_int, c_int, c_int, c_void_p],
    "gibbs_gemm_library_init": [],
    "gibbs_gemm_library": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_long, c_long, c_long, c_void_p],
    "gibbs_argmax": [c_void_p, c_void_p, c_int, c_int, c_long, c_void_p],
    "gibbs_probe_read": [c_void_p, c_long, c_void_p, c_int, c_int, c_void_p],
    "gibbs_repetition_penalty": [c_void_p, c_int, c_int, c_long, c_void_p, c_int, c_void_p, c_void_p, c_void_p],
    "gibbs_sample": [c_void_p, c_void_p, c_int, c_int, c_long, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p],
    "gibbs_linear": [c_void_p, c_long, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "gibbs_skinny_residual_routed": [c_void_p, c_void_p, c_long, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p],
}


_VALUE_SIGNATURES = {
    "gibbs_pair_layout_below_tiles": ([], c_int),
    "gibbs_rule_skinny_splits": ([c_int, c_int, c_int, c_int, c_int], c_int),
    "gibbs_rule_decode_splits": ([c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p], None),
    "gibbs_rule_prefill_splits": ([c_long, c_int, c_int, c_int], c_int),
    "gibbs_rule_prefill_tiles": ([c_int, c_int], c_long),
    "gibbs_rule_prefill_heads": ([c_int, c_int, c_int, c_int, c_int, c_int, c_int], c_int),
    "gibbs_rule_fused_rows": ([], c_int),
    "gibbs_linear_splits": ([c_int, c_int, c_int, c_int, c_long, c_void_p, c_void_p, c_int, c_int, c_int], c_int),
    "gibbs_skinny_residual_workspace": ([c_int, c_int, c_int], c_long),
}


def library() -> ctypes.CDLL:
    """The loaded kernel library (built at the first call if it is not there yet)."""
    global _lib
    if _lib is None:
        with _lock:
            if _lib is None:
                path = _build.ensure_built()
                lib = ctypes.CDLL(path)
                lib.gibbs_last_error.restype = ctypes.c_char_p
                lib.gibbs_abi_version.restype = c_int
                if lib.gibbs_abi_version() != ABI_VERSION:
                    raise KernelError(f"{path} has interface version {lib.gibbs_abi_version()}, expected {ABI_VERSION}")
                for name, argtypes in _SIGNATURES.items():
                    fn = getattr(lib, name)
                    fn.argtypes = argtypes
                    fn.restype = c_int
                for name, (argtypes, restype) in _VALUE_SIGNATURES.items():
                    getattr(lib, name).argtypes, getattr(lib, name).restype = argtypes, restype
                from ..parts import native
                native.declare(lib)
                for name in ("gibbs_gemm_library_timings", "gibbs_gemm_library_plans"):
                    getattr(lib, name).argtypes, getattr(lib, name).restype = [], c_long
                lib.gibbs_attention_decode_workspace.argtypes = [c_int, c_int, c_int, c_int]
                lib.gibbs_attention_decode_workspace.restype = c_long
                _lib = lib
    return _lib


def call(name: str, *args) -> None:
    lib = library()
    status = getattr(lib, name)(*args)
    if status != 0:
        raise KernelError(lib.gibbs_last_error().decode(errors="replace"))


_device_index: Optional[int] = None


def stream() -> int:
    """The current HIP stream of the process's device (one GPU per process), as a raw handle.
    This runs before every launch: the raw query costs a tenth of building a torch Stream object."""
    global _device_index
    if _device_index is None:
        _device_index = torch.cuda.current_device()
    return torch._C._cuda_getCurrentRawStream(_device_index)


def ptr(t: torch.Tensor | None) -> int | None:
    return None if t is None else t.data_ptr()


DTYPE_CODE = {torch.float32: 0, torch.bfloat16: 1}


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return DTYPE_CODE[dtype]
    except KeyError:
        raise KernelError(f"kernels take float32 or bfloat16, not {dtype}") from None


def require_cuda(*tensors: torch.Tensor | None) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise KernelError("kernels take device tensors only; there is no CPU fallback")
