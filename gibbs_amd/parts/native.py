"""The model's step as one native call (csrc/step_plan.hip).

When a model is bound, `NativePlan.build` asks every block to lay its parts down in a native plan
(`emit_native`): weights, sizes and constants go over once, as raw pointers that the parts keep
alive.  A step is then two calls into the library (the bytes of workspace it needs, then the step
itself, which queues every kernel), whatever the number of kernels; stepping through the parts in
Python costs the host about ten microseconds per kernel, which bounds steps of a few dozen to a few
hundred rows.  A model with a part that has no `emit_native` (one registered from outside the
package) simply has no plan and steps through the parts' `forward`, over the same kernels; the two
ways give the same logits bit for bit, and a test holds them against each other.
"""
from __future__ import annotations

import ctypes
from ctypes import c_int, c_long, c_void_p
from typing import List, Optional

import torch

from ..ops import lib as L
from ..ops.lib import KernelError

MAX_GROUPS = 8


class StepArgs(ctypes.Structure):
    """GibbsStepArgs of csrc/step_plan.hip."""
    _fields_ = [("ids", c_void_p), ("pos", c_void_p), ("row_req", c_void_p), ("cu", c_void_p), ("ctx", c_void_p),
                ("slot", c_void_p), ("logit_rows", c_void_p), ("tables", c_void_p * MAX_GROUPS),
                ("widths", c_int * MAX_GROUPS), ("n_rows", c_int), ("n_req", c_int), ("n_logits", c_int),
                ("max_q", c_int), ("max_seq", c_int), ("lead_single", c_int), ("workspace", c_void_p),
                ("workspace_bytes", c_long), ("logits", c_void_p), ("stream", c_void_p), ("x_in", c_void_p),
                ("mirror_in", c_void_p)]


def _ptr(t) -> Optional[int]:
    """Device address of a tensor (or of a packed matrix's tiles), None for None."""
    if t is None:
        return None
    return t.data_ptr()


class PlanBuilder:
    """What parts call from `emit_native`; wraps the library's plan handle."""

    def __init__(self, handle, rt):
        self.handle, self.rt = handle, rt
        self.keep: List = []           # tensors whose addresses the plan holds

    def _call(self, name: str, *args) -> None:
        lib = L.library()
        if getattr(lib, name)(self.handle, *args) != 0:
            raise KernelError(lib.gibbs_last_error().decode(errors="replace"))

    def _held(self, *tensors):
        self.keep += [t for t in tensors if t is not None]
        return [_ptr(t) for t in tensors]

    def block(self, gain1, eps1: float, gain2, eps2: float) -> None:
        g1, g2 = self._held(gain1, gain2)
        self._call("gibbs_plan_add_block", g1, float(eps1), g2, float(eps2))

    def short_conv(self, *, w_in, p_in, w_out, p_out, taps, bias, width: int, kernel: int, state, fusable: bool) -> None:
        assert state.dtype == torch.float32 and state.stride(2) == 1 and state.stride(1) == width
        ptrs = self._held(w_in, p_in, w_out, p_out, taps, bias)
        self.keep.append(state)
        self._call("gibbs_plan_set_conv", *ptrs, int(width), int(kernel), state.data_ptr(), int(state.stride(0)), int(fusable))

    def attention(self, *, w_qkv, p_qkv, w_out, p_out, heads: int, kv_heads: int, head_dim: int, scale: float, window,
                  q_gain, k_gain, qk_eps: float, rotation, kpages, vpages, group: int, owns: bool, fusable: bool) -> None:
        from ..ops import ROPE_VARIANTS
        inv_freq = cos_sin = None
        rot = variant = table_len = 0
        if rotation is not None:
            inv_freq, cos_sin, rot = rotation.inv_freq, rotation.cos_sin, int(rotation.rotary_dim)
            variant = ROPE_VARIANTS[rotation.variant]
            table_len = 0 if cos_sin is None else int(cos_sin.shape[0])
        assert kpages.is_contiguous() and vpages.is_contiguous() and kpages.shape == vpages.shape
        ptrs = self._held(w_qkv, p_qkv, w_out, p_out)
        gains = self._held(q_gain, k_gain)
        tables = self._held(inv_freq, cos_sin)
        self.keep += [kpages, vpages]
        self._call("gibbs_plan_set_attention", *ptrs, int(heads), int(kv_heads), int(head_dim), float(scale), int(window or 0),
                   gains[0], gains[1], float(qk_eps), tables[0], rot, variant, tables[1], table_len, kpages.data_ptr(),
                   vpages.data_ptr(), int(kpages.shape[0]), int(kpages.shape[2]), int(group), int(owns), int(fusable))

    def glu(self, *, w_gate_up, p_gate_up, w_down, p_down, inter: int, activation: int, fusable: bool) -> None:
        ptrs = self._held(w_gate_up, p_gate_up, w_down, p_down)
        self._call("gibbs_plan_set_glu", *ptrs, int(inter), int(activation), int(fusable))


class NativePlan:
    def __init__(self, handle, builder: PlanBuilder, vocab: int, device: torch.device):
        self.handle, self._builder, self.vocab, self.device = handle, builder, vocab, device
        self._arena: Optional[torch.Tensor] = None
        self._args = StepArgs()

    def __del__(self):
        if getattr(self, "handle", None):
            try:
                L.library().gibbs_plan_destroy(self.handle)
            except TypeError:              # (the interpreter is shutting down: the module is gone already)
                pass
            self.handle = None

    @classmethod
    def build(cls, model, views, rt) -> Optional["NativePlan"]:
        """The plan of `model` (bound, with the cache views of its runs), or None if one of its parts
        cannot lay itself down."""
        from ..ops import linear as lin
        if lin.LIBRARY_THROUGH_TORCH:
            return None
        if not hasattr(model.final_norm, "native_norm") or model.final_norm.native_norm() is None:
            return None
        lib = L.library()
        gain, eps = model.final_norm.native_norm()
        handle = lib.gibbs_plan_create(L.dtype_code(rt.act_dtype), model.spec.hidden, model.spec.vocab, model.table.data_ptr(),
                                       L.dtype_code(model.table.dtype), model.head.data_ptr(), _ptr(model.head_packed),
                                       _ptr(gain), float(eps), int(rt.fused_decode_rows), int(not lin.USE_LIBRARY_GEMM))
        if not handle:
            raise KernelError(lib.gibbs_last_error().decode(errors="replace"))
        builder = PlanBuilder(handle, rt)
        builder.keep += [model.table, model.head, model.head_packed, gain]
        plan = cls(handle, builder, model.spec.vocab, rt.device)
        for run, i in enumerate(model.spec.order):
            block = model.blocks[i]
            if not hasattr(block, "emit_native") or not block.emit_native(builder, views[run]):
                return None                    # (the half-built plan is destroyed with `plan`)
        return plan

    # ------------------------------------------------------------------ one step
    def _fill(self, batch, x_in=None, mirror_in=None) -> StepArgs:
        a = self._args
        a.x_in, a.mirror_in = _ptr(x_in), _ptr(mirror_in)
        a.ids, a.pos, a.row_req = batch.ids.data_ptr(), batch.pos.data_ptr(), batch.row_req.data_ptr()
        a.cu, a.ctx, a.slot = batch.cu.data_ptr(), batch.ctx.data_ptr(), batch.slot.data_ptr()
        a.logit_rows = batch.logit_rows.data_ptr() if batch.n_logits else None
        if len(batch.tables) > MAX_GROUPS:
            raise KernelError(f"the native step takes up to {MAX_GROUPS} cache groups")
        for g, t in enumerate(batch.tables):
            a.tables[g], a.widths[g] = t.data_ptr(), int(t.shape[1])
        a.n_rows, a.n_req, a.n_logits = batch.n_rows, batch.n_req, batch.n_logits
        a.max_q, a.max_seq, a.lead_single = batch.max_q, batch.max_seq, batch.lead_single
        a.stream = L.stream()
        return a

    def workspace_bytes(self, batch, x_in=None, mirror_in=None) -> int:
        lib = L.library()
        need = lib.gibbs_plan_workspace(self.handle, ctypes.byref(self._fill(batch, x_in, mirror_in)))
        if need < 0:
            raise KernelError(lib.gibbs_last_error().decode(errors="replace"))
        return int(need)

    def step(self, batch, workspace: Optional[torch.Tensor] = None, x_in: Optional[torch.Tensor] = None,
             mirror_in: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
        """Queues the whole step; returns float32 logits [wanted rows, vocab] (None if none are wanted).
        `workspace`: a byte buffer of the caller's that outlives the step's kernels (a captured graph
        replays over it); default: the plan's own, which grows when a step needs more.  `x_in` (float32
        [rows, hidden]) and `mirror_in` (its bfloat16 copy): the rows' embeddings, when the end of the
        previous step has written them already (the step then starts at its first layer and updates
        them in place)."""
        lib = L.library()
        if x_in is not None:
            assert x_in.dtype == torch.float32 and x_in.is_contiguous() and x_in.shape[0] == batch.n_rows
            assert mirror_in is None or (mirror_in.dtype == torch.bfloat16 and mirror_in.shape == x_in.shape and mirror_in.is_contiguous())
        a = self._fill(batch, x_in, mirror_in)
        need = lib.gibbs_plan_workspace(self.handle, ctypes.byref(a))
        if need < 0:
            raise KernelError(lib.gibbs_last_error().decode(errors="replace"))
        if workspace is None:
            if self._arena is None or self._arena.numel() < need:
                self._arena = None                       # (give the old one back first)
                self._arena = torch.empty(max(int(need * 1.25), 1 << 20), dtype=torch.uint8, device=self.device)
            workspace = self._arena
        elif workspace.numel() < need:
            raise KernelError(f"the step needs {need} bytes of workspace, the caller's buffer has {workspace.numel()}")
        logits = None
        if batch.n_logits:
            logits = torch.empty((batch.n_logits, self.vocab), dtype=torch.float32, device=self.device)
        a.workspace, a.workspace_bytes = workspace.data_ptr(), workspace.numel()
        a.logits = None if logits is None else logits.data_ptr()
        if lib.gibbs_plan_step(self.handle, ctypes.byref(a)) != 0:
            raise KernelError(lib.gibbs_last_error().decode(errors="replace"))
        return logits
