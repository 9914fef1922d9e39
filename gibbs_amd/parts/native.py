"""The model's step as one native call (csrc/step_plan.hip, interface in csrc/step_plan_api.h).

When a model is bound, every block lays its parts down in a `NativePlan` (`Block.emit`): norms and bodies
(mixers, feed-forwards) with their weights, sizes and constants, as raw pointers that the parts keep
alive, and a program of operations that says how the block arranges them.  A step is then one call
into the library, which queues every kernel, whatever their number; every choice of a kernel for a
shape is made there and nowhere else.

Parts that the package brings are native.  A part from elsewhere (a class registered by a test or
another architecture, written with tensor operations) needs nothing but its `forward`: the base
classes lay it down as a callback that the native step calls with the rows it is to read and the
buffer it is to fill.  A part alone (`Mixer.forward`, `Norm.forward`, `Block.forward` of the built-in
parts) runs through a small plan of its own, so it takes the code that a whole step takes.
"""
from __future__ import annotations

import ctypes
from ctypes import CFUNCTYPE, POINTER, c_int, c_long, c_void_p
from typing import Callable, List, Optional

import torch

from ..ops import lib as L
from ..ops.lib import KernelError


class StepArgs(ctypes.Structure):
    """GibbsStepArgs of csrc/step_plan_api.h."""
    _fields_ = [("ids", c_void_p), ("pos", c_void_p), ("row_req", c_void_p), ("cu", c_void_p), ("ctx", c_void_p),
                ("slot", c_void_p), ("logit_rows", c_void_p), ("tables", POINTER(c_void_p)), ("widths", POINTER(c_int)),
                ("n_groups", c_int), ("n_rows", c_int), ("n_req", c_int), ("n_logits", c_int), ("max_q", c_int),
                ("max_seq", c_int), ("lead_single", c_int), ("workspace", c_void_p), ("workspace_bytes", c_long),
                ("logits", c_void_p), ("stream", c_void_p), ("x_in", c_void_p), ("mirror_in", c_void_p),
                ("first_op", c_int), ("n_ops", c_int), ("settle", c_int)]


HOST_BODY = CFUNCTYPE(c_int, c_void_p, POINTER(StepArgs), c_void_p, c_void_p)
HOST_NORM = CFUNCTYPE(c_int, c_void_p, POINTER(StepArgs), c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p)
HOST_ROWS = CFUNCTYPE(c_int, c_void_p, POINTER(StepArgs), c_void_p, c_long)


def _ptr(t) -> Optional[int]:
    """Device address of a tensor (or of a packed matrix's tiles), None for None."""
    return None if t is None else t.data_ptr()


def declare(lib) -> None:
    """Argument and result types of the plan's entry points."""
    P, I, F, LG = c_void_p, c_int, ctypes.c_float, c_long
    sigs = {
        "gibbs_plan_create": ([I, I, I, P, I, P, P, I, I], P),
        "gibbs_plan_destroy": ([P], None),
        "gibbs_plan_norm_rms": ([P, P, F], I),
        "gibbs_plan_norm_host": ([P, HOST_NORM, P], I),
        "gibbs_plan_body_conv": ([P, P, P, P, P, P, P, I, I, P, LG], I),
        "gibbs_plan_body_attention": ([P, P, P, P, P, I, I, I, F, I, P, P, F, P, I, I, P, I, P, P, I, I, I, I, P, HOST_ROWS, P], I),
        "gibbs_plan_body_glu": ([P, P, P, P, P, I, I], I),
        "gibbs_plan_body_host": ([P, HOST_BODY, P, I], I),
        "gibbs_plan_op_half": ([P, I, I], I),
        "gibbs_plan_op_norm": ([P, I], I),
        "gibbs_plan_op_body": ([P, I, I], I),
        "gibbs_plan_op_add": ([P, I], I),
        "gibbs_plan_op_drop": ([P, I], I),
        "gibbs_plan_tail": ([P, I], I),
        "gibbs_plan_op_count": ([P], I),
        "gibbs_plan_workspace": ([P, P], LG),
        "gibbs_plan_step": ([P, P], I),
        "gibbs_plan_last_fused": ([P], I),
        "gibbs_plan_body_forward": ([P, I, P, P, POINTER(LG), POINTER(I)], LG),
        "gibbs_plan_norm_forward": ([P, I, P, P, P, I, P, I, POINTER(LG)], LG),
    }
    for name, (argtypes, restype) in sigs.items():
        fn = getattr(lib, name)
        fn.argtypes, fn.restype = argtypes, restype


class _MinimalBatch:
    """The operands of a part that is run alone without a batch (a feed-forward reads none of them)."""
    def __init__(self, n_rows: int):
        self.n_rows, self.n_req, self.n_logits, self.max_q, self.max_seq, self.lead_single = n_rows, 0, 0, 0, 0, 0
        self.ids = self.pos = self.row_req = self.cu = self.ctx = self.slot = self.logit_rows = None
        self.tables = []


class NativePlan:
    """A plan under construction and, once built, the thing that steps."""

    def __init__(self, rt, hidden: int, vocab: int = 0, table: Optional[torch.Tensor] = None,
                 head: Optional[torch.Tensor] = None, head_packed=None):
        from ..ops import linear as lin
        self.rt, self.hidden, self.vocab, self.device = rt, hidden, vocab, rt.device
        lib = L.library()
        self.handle = lib.gibbs_plan_create(L.dtype_code(rt.act_dtype), int(hidden), int(vocab), _ptr(table),
                                            L.dtype_code(table.dtype) if table is not None else 0, _ptr(head),
                                            _ptr(head_packed), int(rt.fused_decode_rows), int(not lin.USE_LIBRARY_GEMM))
        if not self.handle:
            raise KernelError(lib.gibbs_last_error().decode(errors="replace"))
        self.keep: List = [table, head, head_packed]      # what the plan holds addresses of
        self._callbacks: List = []                         # ctypes thunks must outlive the plan
        self._arena: Optional[torch.Tensor] = None
        self._args = StepArgs()
        self._tables = self._widths = None
        # what a callback finds while a step is being queued
        self.batch = None
        self._workspace: Optional[torch.Tensor] = None
        self._x_in: Optional[torch.Tensor] = None
        self._error: Optional[BaseException] = None

    def __del__(self):
        if getattr(self, "handle", None):
            try:
                L.library().gibbs_plan_destroy(self.handle)
            except TypeError:              # (the interpreter is shutting down: the module is gone already)
                pass
            self.handle = None

    # ------------------------------------------------------------------ building: parts
    def _made(self, index: int) -> int:
        if index < 0:
            raise KernelError(L.library().gibbs_last_error().decode(errors="replace"))
        return index

    def _held(self, *tensors):
        self.keep += [t for t in tensors if t is not None]
        return [_ptr(t) for t in tensors]

    def rms_norm(self, gain: Optional[torch.Tensor], eps: float) -> int:
        (g,) = self._held(gain)
        return self._made(L.library().gibbs_plan_norm_rms(self.handle, g, float(eps)))

    def host_norm(self, forward: Callable) -> int:
        """A norm written with tensor operations: `forward(x, delta, rows, n_rows) -> normed rows` (the
        interface of `Norm.forward`)."""
        def thunk(_user, step, x_ptr, delta_ptr, delta_parts, rows_ptr, n_out, out_ptr):
            try:
                a = step.contents
                x = self._tensor(x_ptr, (a.n_rows, self.hidden), torch.float32)
                delta = None
                if delta_ptr:
                    delta = (self._tensor(delta_ptr, (delta_parts, a.n_rows, self.hidden), torch.float32) if delta_parts >= 2
                             else self._tensor(delta_ptr, (a.n_rows, self.hidden), self.rt.act_dtype))
                rows = self.batch.logit_rows if rows_ptr else None
                out = self._tensor(out_ptr, (n_out, self.hidden), self.rt.act_dtype)
                out.copy_(forward(x, delta, rows, n_out if rows_ptr else None))
                return 0
            except BaseException as exc:            # an exception cannot cross the native frames: it is raised after the call
                self._error = exc
                return 1
        cb = HOST_NORM(thunk)
        self._callbacks.append(cb)
        return self._made(L.library().gibbs_plan_norm_host(self.handle, cb, None))

    def short_conv(self, *, w_in, p_in, w_out, p_out, taps, bias, width: int, kernel: int, state) -> int:
        assert state.dtype == torch.float32 and state.stride(2) == 1 and state.stride(1) == width
        ptrs = self._held(w_in, p_in, w_out, p_out, taps, bias)
        self.keep.append(state)
        return self._made(L.library().gibbs_plan_body_conv(self.handle, *ptrs, int(width), int(kernel), state.data_ptr(),
                                                           int(state.stride(0))))

    def attention(self, *, w_qkv, p_qkv, w_out, p_out, heads: int, kv_heads: int, head_dim: int, scale: float, window,
                  q_gain, k_gain, qk_eps: float, rotation, kpages, vpages, group: int, owns: bool, slopes=None,
                  rows_hook: Optional[Callable] = None) -> int:
        """`rows_hook(q, k, batch)`: changes the step's q [N, heads, head_dim] and k [N, kv_heads, head_dim]
        (None for a mixer that reads another's cache) in place, after the q/k norm and before k is cached."""
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
        (sl,) = self._held(slopes)
        self.keep += [kpages, vpages]
        hook = ctypes.cast(None, HOST_ROWS)
        if rows_hook is not None:
            kv = kv_heads if owns else 0

            def thunk(_user, step, qkv_ptr, ld):
                try:
                    n = step.contents.n_rows
                    rows = self._tensor(qkv_ptr, (n, ld), self.rt.act_dtype)
                    q = rows[:, :heads * head_dim].unflatten(1, (heads, head_dim))
                    k = rows[:, heads * head_dim:(heads + kv) * head_dim].unflatten(1, (kv, head_dim)) if owns else None
                    rows_hook(q, k, self.batch)
                    return 0
                except BaseException as exc:
                    self._error = exc
                    return 1
            hook = HOST_ROWS(thunk)
            self._callbacks.append(hook)
        return self._made(L.library().gibbs_plan_body_attention(
            self.handle, *ptrs, int(heads), int(kv_heads), int(head_dim), float(scale), int(window or 0), gains[0], gains[1],
            float(qk_eps), tables[0], rot, variant, tables[1], table_len, kpages.data_ptr(), vpages.data_ptr(),
            int(kpages.shape[0]), int(kpages.shape[2]), int(group), int(owns), sl, hook, None))

    def glu(self, *, w_gate_up, p_gate_up, w_down, p_down, inter: int, activation: int) -> int:
        ptrs = self._held(w_gate_up, p_gate_up, w_down, p_down)
        return self._made(L.library().gibbs_plan_body_glu(self.handle, *ptrs, int(inter), int(activation)))

    def host_body(self, forward: Callable, group: Optional[int] = None) -> int:
        """A mixer or feed-forward written with tensor operations: `forward(h, batch) -> delta [N, hidden]`
        (or float32 partial sums [S, N, hidden]).  `group`: the cache group whose block table it reads."""
        def thunk(_user, step, h_ptr, out_ptr):
            try:
                n = step.contents.n_rows
                h = self._tensor(h_ptr, (n, self.hidden), self.rt.act_dtype)
                out = self._tensor(out_ptr, (n, self.hidden), self.rt.act_dtype)
                delta = forward(h, self.batch)
                out.copy_(delta.sum(0) if delta.dim() == 3 else delta)
                return 0
            except BaseException as exc:
                self._error = exc
                return 1
        cb = HOST_BODY(thunk)
        self._callbacks.append(cb)
        return self._made(L.library().gibbs_plan_body_host(self.handle, cb, None, -1 if group is None else int(group)))

    # ------------------------------------------------------------------ building: the program
    def half(self, norm: int, body: int) -> None:
        """x += body(norm(x)); in fused decode kernels where the step, the norm and the body allow them."""
        self._made(L.library().gibbs_plan_op_half(self.handle, norm, body))

    def normed(self, norm: int) -> int:
        """-> value: norm(x + what is pending)."""
        return self._made(L.library().gibbs_plan_op_norm(self.handle, norm))

    def apply(self, body: int, value: int) -> int:
        """-> value: body(normed rows)."""
        return self._made(L.library().gibbs_plan_op_body(self.handle, body, value))

    def add(self, value: int) -> None:
        """x += delta (it stays pending until the next norm reads x, which adds it on the way)."""
        self._made(L.library().gibbs_plan_op_add(self.handle, value))

    def drop(self, value: int) -> None:
        self._made(L.library().gibbs_plan_op_drop(self.handle, value))

    def tail(self, norm: int) -> None:
        self._made(L.library().gibbs_plan_tail(self.handle, norm))

    def op_count(self) -> int:
        return int(L.library().gibbs_plan_op_count(self.handle))

    @classmethod
    def build(cls, model, views, rt) -> "NativePlan":
        """The plan of a bound `DecoderModel` (`views[run]`: the cache views of the run's mixers by role)."""
        plan = cls(rt, model.spec.hidden, model.spec.vocab, model.table, model.head, model.head_packed)
        for run, i in enumerate(model.spec.order):
            model.blocks[i].emit(plan, views[run])
        plan.tail(model.final_norm.emit(plan))
        return plan

    # ------------------------------------------------------------------ running
    def _tensor(self, ptr: int, shape, dtype: torch.dtype) -> torch.Tensor:
        """The tensor behind a pointer that the native step hands to a callback: a piece of the step's
        workspace, or the caller's own residual rows."""
        n = 1
        for s in shape:
            n *= s
        nbytes = n * torch.empty((), dtype=dtype).element_size()
        for base in (self._workspace, self._x_in):
            if base is None:
                continue
            off = ptr - base.data_ptr()
            if 0 <= off and off + nbytes <= base.numel() * base.element_size():
                return base.view(-1).view(torch.uint8)[off:off + nbytes].view(dtype).view(*shape)
        raise KernelError("a callback of the native step was handed memory that is neither the workspace nor the caller's rows")

    def _fill(self, batch, x_in=None, mirror_in=None, first_op: int = 0, n_ops: int = 0, settle: bool = False) -> StepArgs:
        a = self._args
        a.x_in, a.mirror_in = _ptr(x_in), _ptr(mirror_in)
        a.ids, a.pos, a.row_req = _ptr(batch.ids), _ptr(batch.pos), _ptr(batch.row_req)
        a.cu, a.ctx, a.slot = _ptr(batch.cu), _ptr(batch.ctx), _ptr(batch.slot)
        a.logit_rows = _ptr(batch.logit_rows) if batch.n_logits else None
        g = len(batch.tables)
        if self._tables is None or len(self._tables) != max(g, 1):
            self._tables, self._widths = (c_void_p * max(g, 1))(), (c_int * max(g, 1))()
        for i, t in enumerate(batch.tables):
            self._tables[i], self._widths[i] = t.data_ptr(), int(t.shape[1])
        a.tables, a.widths, a.n_groups = self._tables, self._widths, g
        a.n_rows, a.n_req, a.n_logits = batch.n_rows, batch.n_req, batch.n_logits
        a.max_q, a.max_seq, a.lead_single = batch.max_q, batch.max_seq, batch.lead_single
        a.first_op, a.n_ops, a.settle = first_op, n_ops, int(settle)
        a.workspace, a.workspace_bytes, a.logits = None, 0, None
        a.stream = L.stream()
        return a

    def _raise(self):
        exc, self._error = self._error, None
        if exc is not None:
            raise exc
        raise KernelError(L.library().gibbs_last_error().decode(errors="replace"))

    def _own_workspace(self, need: int) -> torch.Tensor:
        if self._arena is None or self._arena.numel() < need:
            self._arena = None                       # (give the old one back first)
            self._arena = torch.empty(max(int(need * 1.25), 1 << 20), dtype=torch.uint8, device=self.device)
        return self._arena

    def workspace_bytes(self, batch, x_in=None, mirror_in=None) -> int:
        need = L.library().gibbs_plan_workspace(self.handle, ctypes.byref(self._fill(batch, x_in, mirror_in)))
        if need < 0:
            self._raise()
        return int(need)

    def step(self, batch, workspace: Optional[torch.Tensor] = None, x_in: Optional[torch.Tensor] = None,
             mirror_in: Optional[torch.Tensor] = None, first_op: int = 0, n_ops: int = 0,
             settle: bool = False) -> Optional[torch.Tensor]:
        """Queues the whole step; returns float32 logits [wanted rows, vocab] (None if none are wanted).
        `workspace`: a byte buffer of the caller's that outlives the step's kernels (a captured graph
        replays over it); default: the plan's own, which grows when a step needs more.  `x_in` (float32
        [rows, hidden]) and `mirror_in` (its bfloat16 copy): the rows' embeddings, when the end of the
        previous step has written them already (the step then starts at its first layer and updates
        them in place).  `first_op`, `n_ops`: only these operations of the program run (no logits then);
        `settle`: whatever delta is still pending at the end is added into x."""
        lib = L.library()
        if x_in is not None:
            assert x_in.dtype == torch.float32 and x_in.is_contiguous() and x_in.shape[0] == batch.n_rows
            assert mirror_in is None or (mirror_in.dtype == torch.bfloat16 and mirror_in.shape == x_in.shape and mirror_in.is_contiguous())
        a = self._fill(batch, x_in, mirror_in, first_op, n_ops, settle)
        need = lib.gibbs_plan_workspace(self.handle, ctypes.byref(a))
        if need < 0:
            self._raise()
        if workspace is None:
            workspace = self._own_workspace(need)
        elif workspace.numel() < need:
            raise KernelError(f"the step needs {need} bytes of workspace, the caller's buffer has {workspace.numel()}")
        logits = None
        if batch.n_logits and n_ops == 0:
            logits = torch.empty((batch.n_logits, self.vocab), dtype=torch.float32, device=self.device)
        a.workspace, a.workspace_bytes = workspace.data_ptr(), workspace.numel()
        a.logits = None if logits is None else logits.data_ptr()
        self.batch, self._workspace, self._x_in = batch, workspace, x_in
        try:
            if lib.gibbs_plan_step(self.handle, ctypes.byref(a)) != 0:
                self._raise()
        finally:
            self.batch = self._workspace = self._x_in = None
        return logits

    def last_fused(self) -> int:
        """Halves of the last step that ran as fused decode kernels."""
        return int(L.library().gibbs_plan_last_fused(self.handle))

    # ------------------------------------------------------------------ one part alone
    def body_forward(self, body: int, h: torch.Tensor, batch) -> torch.Tensor:
        """delta of the normed rows `h` by body number `body`: [N, hidden], or float32 partial sums [S, N, hidden]."""
        lib = L.library()
        assert h.is_contiguous() and h.dtype == self.rt.act_dtype and h.shape[1] == self.hidden
        batch = _MinimalBatch(h.shape[0]) if batch is None else batch
        a = self._fill(batch)
        a.n_rows = h.shape[0]
        off, parts = c_long(0), c_int(0)
        need = lib.gibbs_plan_body_forward(self.handle, body, ctypes.byref(a), h.data_ptr(), ctypes.byref(off), ctypes.byref(parts))
        if need < 0:
            self._raise()
        workspace = torch.empty(max(int(need), 256), dtype=torch.uint8, device=self.device)   # (the result lives in it)
        a.workspace, a.workspace_bytes = workspace.data_ptr(), workspace.numel()
        self.batch, self._workspace = batch, workspace
        try:
            if lib.gibbs_plan_body_forward(self.handle, body, ctypes.byref(a), h.data_ptr(), ctypes.byref(off), ctypes.byref(parts)) != 0:
                self._raise()
        finally:
            self.batch = self._workspace = None
        n = h.shape[0]
        if parts.value >= 2:
            return workspace[off.value:off.value + parts.value * n * self.hidden * 4].view(torch.float32).view(parts.value, n, self.hidden)
        size = torch.empty((), dtype=self.rt.act_dtype).element_size()
        return workspace[off.value:off.value + n * self.hidden * size].view(self.rt.act_dtype).view(n, self.hidden)

    def norm_forward(self, norm: int, x: torch.Tensor, delta: Optional[torch.Tensor], rows: Optional[torch.Tensor],
                     n_rows: Optional[int]) -> torch.Tensor:
        lib = L.library()
        assert x.dtype == torch.float32 and x.is_contiguous() and x.shape[1] == self.hidden
        parts = 0
        if delta is not None:
            assert delta.is_contiguous()
            if delta.dim() == 3:
                assert delta.dtype == torch.float32 and delta.shape[1:] == x.shape
                parts = delta.shape[0]
            else:
                assert delta.shape == x.shape and delta.dtype == self.rt.act_dtype
                parts = 1
        n_out = x.shape[0] if rows is None else (rows.numel() if n_rows is None else n_rows)
        a = self._fill(_MinimalBatch(x.shape[0]))
        off = c_long(0)
        call = lambda: lib.gibbs_plan_norm_forward(self.handle, norm, ctypes.byref(a), x.data_ptr(), _ptr(delta), parts,
                                                   _ptr(rows), int(n_out), ctypes.byref(off))
        need = call()
        if need < 0:
            self._raise()
        workspace = torch.empty(max(int(need), 256), dtype=torch.uint8, device=self.device)
        a.workspace, a.workspace_bytes = workspace.data_ptr(), workspace.numel()
        if call() != 0:
            self._raise()
        size = torch.empty((), dtype=self.rt.act_dtype).element_size()
        return workspace[off.value:off.value + n_out * self.hidden * size].view(self.rt.act_dtype).view(n_out, self.hidden)
