"""Python entry points of the HIP kernels: each checks on the host that operand shapes match
what the kernel and its grid assume, then queues the kernel on the current stream."""
from __future__ import annotations

from typing import Optional

import torch

from .lib import KernelError, call, dtype_code, library, ptr, require_cuda, stream

ROPE_VARIANTS = {"half_split": 0, "interleaved": 1}
ACTIVATIONS = {"silu": 0, "gelu_tanh": 1, "gelu": 2, "relu": 3}     # csrc/activation.h


def _i32(t: torch.Tensor, n: int, what: str) -> None:
    if t.dtype != torch.int32 or not t.is_contiguous() or t.numel() < n:
        raise KernelError(f"{what} must be a contiguous int32 tensor of at least {n} elements")


def embed(table: torch.Tensor, ids: torch.Tensor, n: int, out: Optional[torch.Tensor] = None,
          mirror: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x[n, :] = float32(table[ids[n], :]); `mirror` (optional, bfloat16 [n, hidden]) gets the same rows."""
    require_cuda(table, ids)
    vocab, hidden = table.shape
    _i32(ids, n, "ids")
    if out is None:
        out = torch.empty((n, hidden), dtype=torch.float32, device=table.device)
    assert out.dtype == torch.float32 and out.is_contiguous() and out.shape == (n, hidden)
    assert table.is_contiguous()
    if mirror is not None:
        assert mirror.dtype == torch.bfloat16 and mirror.shape == (n, hidden) and mirror.is_contiguous()
    call("gibbs_embed", ptr(table), dtype_code(table.dtype), ptr(ids), ptr(out), ptr(mirror), n, hidden, vocab, stream())
    return out


def add_rmsnorm(x: torch.Tensor, delta: Optional[torch.Tensor], gain: Optional[torch.Tensor], eps: float,
                out_dtype: torch.dtype, rows: Optional[torch.Tensor] = None, n_out: Optional[int] = None,
                out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """v = x (+ delta); x <- v when all rows are normed; out = v * rsqrt(mean(v^2) + eps) * gain.
    With `rows`, only those rows are normed (and x is left as it is).  `delta` is [N, H] in the
    output dtype, or float32 [S, N, H]: partial sums that are added in ascending s."""
    require_cuda(x, delta, gain, rows)
    n, hidden = x.shape
    assert x.dtype == torch.float32 and x.is_contiguous()
    assert gain is None or (gain.dtype == torch.float32 and gain.shape == (hidden,) and gain.is_contiguous())
    partials = delta is not None and delta.dim() == 3
    if partials:
        assert delta.dtype == torch.float32 and delta.shape[1:] == x.shape and delta.is_contiguous()
    elif delta is not None:
        assert delta.shape == x.shape and delta.dtype == out_dtype and delta.is_contiguous()
    if rows is None:
        n_out = n
    else:
        n_out = rows.numel() if n_out is None else n_out
        _i32(rows, n_out, "rows")
    if out is None:
        out = torch.empty((n_out, hidden), dtype=out_dtype, device=x.device)
    assert out.shape == (n_out, hidden) and out.dtype == out_dtype and out.is_contiguous()
    if partials:
        call("gibbs_add_partials_rmsnorm", ptr(x), ptr(delta), delta.shape[0], delta.stride(0), ptr(gain), float(eps),
             ptr(out), dtype_code(out_dtype), ptr(rows), n_out, hidden, stream())
        return out
    call("gibbs_add_rmsnorm", ptr(x), ptr(delta), ptr(gain), float(eps), ptr(out), dtype_code(out_dtype),
         ptr(rows), n_out, hidden, stream())
    return out


def residual_add(x: torch.Tensor, delta: Optional[torch.Tensor], mirror: Optional[torch.Tensor] = None) -> None:
    """x += delta (if given; float32 parts [S, N, H] are added in ascending s); `mirror` (optional,
    bfloat16, same shape as x) = bfloat16(x)."""
    require_cuda(x, delta, mirror)
    assert x.dtype == torch.float32 and x.is_contiguous()
    parts = 1
    if delta is not None:
        assert delta.is_contiguous()
        if delta.dim() == 3:
            assert delta.dtype == torch.float32 and delta.shape[1:] == x.shape
            parts = delta.shape[0]
        else:
            assert delta.shape == x.shape
    if mirror is not None:
        assert mirror.dtype == torch.bfloat16 and mirror.shape == x.shape and mirror.is_contiguous()
    call("gibbs_residual_add", ptr(x), ptr(delta), dtype_code(delta.dtype) if delta is not None else 0, parts,
         x.numel(), ptr(mirror), x.numel(), stream())


def gemm_f32(a: torch.Tensor, w: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[n, o] = sum_k a[n, k] * w[o, k], all float32, plain FMA."""
    require_cuda(a, w)
    assert a.dtype == torch.float32 and w.dtype == torch.float32
    assert a.dim() == 2 and w.dim() == 2 and a.shape[1] == w.shape[1], (a.shape, w.shape)
    assert a.stride(1) == 1 and w.stride(1) == 1
    n, i = a.shape
    o = w.shape[0]
    if out is None:
        out = torch.empty((n, o), dtype=torch.float32, device=a.device)
    assert out.shape == (n, o) and out.dtype == torch.float32 and out.stride(1) == 1
    call("gibbs_gemm_f32", ptr(a), ptr(w), ptr(out), n, o, i, a.stride(0) if n > 1 else i,
         w.stride(0), out.stride(0) if n > 1 else o, stream())
    return out


def gemm_bf16_plain(a: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """The bfloat16 product for shapes the matrix-core kernels refuse (inner size or row strides
    that are no multiple of 8): plain FMA, float32 accumulation."""
    require_cuda(a, w)
    assert a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16
    assert a.dim() == 2 and w.dim() == 2 and a.shape[1] == w.shape[1] and a.stride(1) == 1 and w.stride(1) == 1
    n, i = a.shape
    o = w.shape[0]
    out = torch.empty((n, o), dtype=out_dtype, device=a.device)
    call("gibbs_gemm_bf16_plain", ptr(a), ptr(w), ptr(out), dtype_code(out_dtype), n, o, i,
         a.stride(0) if n > 1 else i, w.stride(0), o, stream())
    return out


def gemm_bf16(a: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16,
              out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[n, o] = sum_k a[n, k] * w[o, k]: bfloat16 operands on the matrix cores, float32
    accumulation, bfloat16 or float32 output."""
    require_cuda(a, w)
    assert a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16
    assert a.dim() == 2 and w.dim() == 2 and a.shape[1] == w.shape[1], (a.shape, w.shape)
    assert a.stride(1) == 1 and w.stride(1) == 1
    n, i = a.shape
    o = w.shape[0]
    lda = a.stride(0) if n > 1 else i
    if i % 8 or lda % 8 or w.stride(0) % 8:
        raise KernelError(f"gemm_bf16: inner size {i} and row strides must be multiples of 8")
    if out is None:
        out = torch.empty((n, o), dtype=out_dtype, device=a.device)
    assert out.shape == (n, o) and out.dtype == out_dtype and out.stride(1) == 1
    call("gibbs_gemm_bf16", ptr(a), ptr(w), ptr(out), dtype_code(out_dtype), n, o, i, lda, w.stride(0),
         out.stride(0) if n > 1 else o, stream())
    return out


_library_ready = False


def gemm_library(a: torch.Tensor, w: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[n, o] = sum_k a[n, k] * w[o, k] by the library (hipBLASLt called directly, its choice of
    algorithm kept per shape): bfloat16 operands and output, float32 accumulation."""
    global _library_ready
    require_cuda(a, w)
    assert a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16
    assert a.dim() == 2 and w.dim() == 2 and a.shape[1] == w.shape[1], (a.shape, w.shape)
    assert a.stride(1) == 1 and w.stride(1) == 1
    n, i = a.shape
    o = w.shape[0]
    if out is None:
        out = torch.empty((n, o), dtype=torch.bfloat16, device=a.device)
    assert out.shape == (n, o) and out.dtype == torch.bfloat16 and out.stride(1) == 1
    if not _library_ready:
        call("gibbs_gemm_library_init")
        _library_ready = True
    call("gibbs_gemm_library", ptr(a), ptr(w), ptr(out), n, o, i, a.stride(0) if n > 1 else i, w.stride(0),
         out.stride(0) if n > 1 else o, stream())
    return out


def one_off_work() -> int:
    """A count that grows whenever a call did set-up work that its like will not do again (the timed
    choice of a library algorithm for a new shape): a step during which it grew is no measure of
    what such steps cost."""
    return int(library().gibbs_gemm_library_timings())


def pair_layout(rows: int) -> bool:
    """Whether a packed matrix of `rows` rows (per row group) is in the pair layout; the rule is the library's."""
    return -(-rows // 16) < library().gibbs_pair_layout_below_tiles()


class PackedWeight:
    """A matrix [groups * rows, inner] (bfloat16) in the order the few-row products read it, each row group
    by itself, zeros beyond rows and inner.  A wave's load of an MFMA A operand is then 1 KB of consecutive
    memory (8 requests of 128 bytes instead of 16 of 64), which is worth a fifth of the time of a
    weight-streaming product.  Two orders (csrc/packed_layout.h), chosen by the rows of a group:
    16-row tiles, [group][ceil(rows/16)][ceil(inner/32)][64 lanes][8], lane (r, g) of a tile holding
    W[tile row * 16 + r][k tile * 32 + g * 8 .. + 8]; and, for matrices of so few rows that workgroups take 8
    features each, 8-row tiles of two k tiles, [group][2 ceil(rows/16)][ceil(inner/64)][g][half][r8][8] with
    W[tile * 8 + r8][pair * 64 + half * 32 + g * 8 .. + 8].  `shape`, `dtype` and `stride(0) == 0` let it stand
    where the row-major matrix does."""

    def __init__(self, w: torch.Tensor, groups: int = 1):
        assert w.dim() == 2 and w.dtype == torch.bfloat16 and w.shape[0] % groups == 0
        total, inner = w.shape
        rows = total // groups
        self.pairs = pair_layout(rows)
        rows_p = -(-rows // 16) * 16
        inner_p = -(-inner // 64) * 64 if self.pairs else -(-inner // 32) * 32
        padded = torch.zeros((groups, rows_p, inner_p), dtype=w.dtype, device=w.device)
        padded[:, :rows, :inner] = w.reshape(groups, rows, inner)
        if self.pairs:
            tiles = padded.view(groups, rows_p // 8, 8, inner_p // 64, 2, 4, 8).permute(0, 1, 3, 5, 4, 2, 6)
        else:
            tiles = padded.view(groups, rows_p // 16, 16, inner_p // 32, 4, 8).permute(0, 1, 3, 4, 2, 5)
        self.data = tiles.contiguous()                     # [group][row tile][k tile or pair][g]([half])[r][8]
        self.shape, self.dtype, self.groups, self.device = (total, inner), w.dtype, groups, w.device

    def dim(self) -> int:
        return 2

    def stride(self, d: int) -> int:
        return 0 if d == 0 else 1

    def data_ptr(self) -> int:
        return self.data.data_ptr()

    @property
    def is_cuda(self) -> bool:
        return self.data.is_cuda


def _w(w) -> torch.Tensor:
    """The tensor behind a weight operand (a row-major matrix, or a PackedWeight's tiles)."""
    return w.data if isinstance(w, PackedWeight) else w


def skinny_splits(n_out: int, inner: int, want_blocks: int = 512, features: int = 16, min_k: int = 1024) -> int:
    """How many ranges of k `gemm_skinny` should cut a product into so that at least `want_blocks`
    workgroups run (a workgroup owns `features` output features), each with at least `min_k` of k
    (the rule is the native step's)."""
    return int(library().gibbs_rule_skinny_splits(n_out, inner, want_blocks, features, min_k))


def gemm_skinny(x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16, k_splits: int = 1,
                out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """y = x @ w^T for at most 64 rows of x, streaming w once.  k_splits > 1 returns float32
    partial sums [k_splits, N, O] (ranges of k) for the consumer to add.  `w` may be a PackedWeight."""
    require_cuda(x, _w(w))
    if isinstance(w, PackedWeight) and w.groups != 1:
        raise KernelError("gemm_skinny: the weights are packed in row groups")
    assert x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16
    assert x.dim() == 2 and w.dim() == 2 and x.shape[1] == w.shape[1], (x.shape, w.shape)
    assert x.stride(1) == 1 and w.stride(1) == 1
    n, i = x.shape
    o = w.shape[0]
    if not 1 <= n <= 64:
        raise KernelError(f"gemm_skinny takes 1..64 rows, not {n}")
    ldx = x.stride(0) if n > 1 else i
    if i % 8 or ldx % 8 or w.stride(0) % 8:
        raise KernelError(f"gemm_skinny: inner size {i} and row strides must be multiples of 8")
    if k_splits > 1:
        out_dtype = torch.float32
        shape = (k_splits, n, o)
    else:
        shape = (n, o)
    if out is None:
        out = torch.empty(shape, dtype=out_dtype, device=x.device)
    assert out.shape == shape and out.dtype == out_dtype and out.is_contiguous()
    call("gibbs_gemm_skinny", ptr(x), ptr(_w(w)), ptr(out), dtype_code(out_dtype), n, o, i, ldx, w.stride(0), o, k_splits,
         stream())
    return out


def _skinny_check(x: torch.Tensor, w, what: str, groups: int = 1) -> tuple[int, int, int]:
    require_cuda(x, _w(w))
    if isinstance(w, PackedWeight) and w.groups != groups:
        raise KernelError(f"{what}: the weights are packed in {w.groups} row groups, the product reads {groups}")
    assert x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and x.dim() == 2 and w.dim() == 2
    assert x.shape[1] == w.shape[1] and x.stride(1) == 1 and w.stride(1) == 1, (x.shape, w.shape)
    n, i = x.shape
    if not 1 <= n <= 64:
        raise KernelError(f"{what} takes 1..64 rows, not {n}")
    ldx = x.stride(0) if n > 1 else i
    if i % 8 or ldx % 8 or w.stride(0) % 8:
        raise KernelError(f"{what}: inner size {i} and row strides must be multiples of 8")
    return n, i, ldx


def skinny_store(x: torch.Tensor, w: torch.Tensor, rms_eps: Optional[float] = None,
                 out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """y = s * (x @ w^T), bfloat16, for at most 64 rows; with `rms_eps` the rows of x are the raw
    residual stream and s_n = 1/sqrt(mean(x_n^2) + eps) (the norm's gain being folded into w)."""
    n, i, ldx = _skinny_check(x, w, "skinny_store")
    o = w.shape[0]
    if out is None:
        out = torch.empty((n, o), dtype=torch.bfloat16, device=x.device)
    assert out.shape == (n, o) and out.dtype == torch.bfloat16 and out.is_contiguous()
    call("gibbs_skinny_store", ptr(x), ptr(_w(w)), ptr(out), n, o, i, ldx, w.stride(0), o, int(rms_eps is not None),
         float(rms_eps or 0.0), stream())
    return out


def skinny_residual(x_in: torch.Tensor, w: torch.Tensor, stream_x: torch.Tensor, mirror: torch.Tensor) -> None:
    """stream_x += x_in @ w^T (float32 residual stream, in place); mirror = bfloat16(stream_x)."""
    n, i, ldx = _skinny_check(x_in, w, "skinny_residual")
    o = w.shape[0]
    assert stream_x.dtype == torch.float32 and stream_x.shape == (n, o) and stream_x.is_contiguous()
    assert mirror.dtype == torch.bfloat16 and mirror.shape == (n, o) and mirror.is_contiguous()
    # (many rows and a long inner size: k is cut over workgroups and the float32 partial sums are added to the
    # stream by a second kernel; whether, and into how many, is the native step's rule)
    floats = int(library().gibbs_skinny_residual_workspace(n, o, i))
    parts = torch.empty(floats, dtype=torch.float32, device=x_in.device) if floats else None
    call("gibbs_skinny_residual_routed", ptr(x_in), ptr(_w(w)), w.stride(0), ptr(stream_x), ptr(mirror), n, o, i, ptr(parts), stream())


def skinny_glu(x: torch.Tensor, w_gate_up: torch.Tensor, rms_eps: Optional[float] = None,
               out: Optional[torch.Tensor] = None, activation: str = "silu") -> torch.Tensor:
    """out = act(s x @ gate^T) * (s x @ up^T) with w_gate_up = [gate rows; up rows]."""
    n, i, ldx = _skinny_check(x, w_gate_up, "skinny_glu", groups=2)
    if activation not in ACTIVATIONS:
        raise KernelError(f"skinny_glu: activation {activation!r} is not implemented; known: {sorted(ACTIVATIONS)}")
    assert w_gate_up.shape[0] % 2 == 0
    f = w_gate_up.shape[0] // 2
    if out is None:
        out = torch.empty((n, f), dtype=torch.bfloat16, device=x.device)
    assert out.shape == (n, f) and out.dtype == torch.bfloat16 and out.is_contiguous()
    call("gibbs_skinny_glu", ptr(x), ptr(_w(w_gate_up)), ptr(out), n, f, i, ldx, w_gate_up.stride(0), f,
         int(rms_eps is not None), float(rms_eps or 0.0), ACTIVATIONS[activation], stream())
    return out


def skinny_conv(x: torch.Tensor, w_in: torch.Tensor, taps: torch.Tensor, bias: Optional[torch.Tensor],
                state: torch.Tensor, slot: torch.Tensor, ctx: torch.Tensor, rms_eps: Optional[float] = None,
                out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """In-projection and gated short convolution for a step of decoded tokens (row n is one token of
    the request in slot[n] with ctx[n] cached positions): w_in = [B rows; C rows; x rows]."""
    n, i, ldx = _skinny_check(x, w_in, "skinny_conv", groups=3)
    require_cuda(taps, bias, state, slot, ctx)
    c, k = taps.shape
    assert w_in.shape[0] == 3 * c
    assert taps.dtype == torch.float32 and taps.is_contiguous()
    assert bias is None or (bias.dtype == torch.float32 and bias.shape == (c,) and bias.is_contiguous())
    assert state.dtype == torch.float32 and state.shape[1:] == (k - 1, c) and state.stride(2) == 1 and state.stride(1) == c
    _i32(slot, n, "slot"); _i32(ctx, n, "ctx")
    if not 2 <= k <= 8:
        raise KernelError(f"skinny_conv: kernel length {k} outside 2..8")
    if out is None:
        out = torch.empty((n, c), dtype=torch.bfloat16, device=x.device)
    assert out.shape == (n, c) and out.dtype == torch.bfloat16 and out.is_contiguous()
    call("gibbs_skinny_conv", ptr(x), ptr(_w(w_in)), ptr(out), n, c, i, ldx, w_in.stride(0), int(rms_eps is not None),
         float(rms_eps or 0.0), ptr(taps), ptr(bias), ptr(state), state.stride(0), ptr(slot), ptr(ctx), k, stream())
    return out


def attention_decode_fused(qkv: torch.Tensor, n_rows: int, nh: int, nkv: int, hd: int, kpages: torch.Tensor,
                           vpages: torch.Tensor, table: torch.Tensor, n_req: int, pos: torch.Tensor,
                           row_req: Optional[torch.Tensor], scale: float, *, q_gain: Optional[torch.Tensor],
                           k_gain: Optional[torch.Tensor], eps: float, inv_freq: Optional[torch.Tensor],
                           rotary_dim: int, variant: str, window: Optional[int] = None,
                           max_seq: int = 0, n_splits: Optional[int] = None,
                           out: Optional[torch.Tensor] = None, cos_sin: Optional[torch.Tensor] = None,
                           waves: Optional[int] = None, kind: str = "auto") -> torch.Tensor:
    """Decode attention straight from the raw fused projection qkv[N, (nh + 2 nkv) hd] of N decoded
    tokens: q/k norm and rotation, the write of the new key and value to their pages, attention over
    split keys in one kernel (followed by the merge of the slices).  `cos_sin` as in `qk_rope_kv`."""
    require_cuda(qkv, kpages, vpages, table, pos, row_req, q_gain, k_gain, inv_freq, cos_sin)
    table_len = _check_cos_sin(cos_sin, inv_freq, rotary_dim)
    if qkv.dtype != torch.bfloat16:
        raise KernelError("attention_decode_fused is a bfloat16 kernel")
    if hd % 16 or hd > 256:
        raise KernelError(f"attention_decode_fused: head size {hd} must be a multiple of 16 up to 256")
    assert qkv.dim() == 2 and qkv.shape[0] == n_rows and qkv.stride(1) == 1 and qkv.shape[1] >= (nh + 2 * nkv) * hd
    num_pages, page_size = _check_pages(kpages, nkv, hd, qkv.dtype)
    assert _check_pages(vpages, nkv, hd, qkv.dtype) == (num_pages, page_size)
    assert table.dim() == 2 and table.shape[0] >= n_req
    _i32(table, n_req, "block table"); _i32(pos, n_rows, "pos")
    if row_req is not None:   # (None: row n is request n)
        _i32(row_req, n_rows, "row_req")
    else:
        assert n_rows <= table.shape[0], "rows without a row-to-request map are requests"
    for g in (q_gain, k_gain):
        assert g is None or (g.dtype == torch.float32 and g.shape == (hd,) and g.is_contiguous())
    if inv_freq is not None:
        assert inv_freq.dtype == torch.float32 and inv_freq.shape == (rotary_dim // 2,) and inv_freq.is_contiguous()
        if rotary_dim % 16:
            raise KernelError(f"attention_decode_fused: rotary_dim {rotary_dim} must be a multiple of 16")
    if n_splits is None or waves is None:
        auto_splits, auto_waves = decode_splits(n_rows, nkv, nh // nkv, max_seq, hd, kind, page_size)
        n_splits = auto_splits if n_splits is None else n_splits
        waves = auto_waves if waves is None else waves
    partial = None
    if n_splits > 1:
        partial = torch.empty(slices_workspace(n_rows, nh, hd, n_splits), dtype=torch.float32, device=qkv.device)
    if out is None:
        out = torch.empty((n_rows, nh * hd), dtype=qkv.dtype, device=qkv.device)
    assert out.shape == (n_rows, nh * hd) and out.dtype == qkv.dtype and out.is_contiguous()
    call("gibbs_attention_decode_fused", ptr(qkv), ptr(kpages), ptr(vpages), ptr(out), ptr(partial),
         ptr(q_gain), ptr(k_gain), float(eps), ptr(inv_freq), rotary_dim, ROPE_VARIANTS[variant], ptr(cos_sin),
         table_len, ptr(pos), ptr(row_req), ptr(table), table.shape[1], page_size, num_pages, n_rows, nh, nkv, hd,
         qkv.stride(0) if n_rows > 1 else qkv.shape[1], nh * hd, float(scale), int(window or 0), n_splits, int(waves),
         DECODE_KINDS[kind], int(max_seq), stream())
    return out


def glu(gu: torch.Tensor, activation: str = "silu", out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[n, f] = act(gu[n, f]) * gu[n, F + f]."""
    require_cuda(gu)
    n, two_f = gu.shape
    assert two_f % 2 == 0 and gu.is_contiguous()
    if activation not in ACTIVATIONS:
        raise KernelError(f"glu: activation {activation!r} is not implemented; known: {sorted(ACTIVATIONS)}")
    f = two_f // 2
    if out is None:
        out = torch.empty((n, f), dtype=gu.dtype, device=gu.device)
    assert out.shape == (n, f) and out.dtype == gu.dtype and out.is_contiguous()
    call("gibbs_glu", ptr(gu), ptr(out), dtype_code(gu.dtype), n, f, ACTIVATIONS[activation], stream())
    return out


def shortconv(bcx: torch.Tensor, taps: torch.Tensor, bias: Optional[torch.Tensor], state: torch.Tensor,
              cu: torch.Tensor, ctx: torch.Tensor, slot: torch.Tensor, n_rows: int, n_req: int,
              out: Optional[torch.Tensor] = None, lead_single: Optional[int] = None) -> torch.Tensor:
    """Gated short convolution of a ragged batch with its per-request state.
    bcx: [N, 3C]; taps: [C, K] float32; state: [slots, K-1, C] float32 (slot stride free).
    lead_single: how many requests at the head of the batch bring exactly one row each (the kernel finds their
    rows without a walk over the requests); None: all of them if there are as many rows as requests, else none."""
    require_cuda(bcx, taps, bias, state, cu, ctx, slot)
    c, k = taps.shape
    assert bcx.shape == (n_rows, 3 * c) and bcx.is_contiguous()
    assert taps.dtype == torch.float32 and taps.is_contiguous()
    assert bias is None or (bias.dtype == torch.float32 and bias.shape == (c,) and bias.is_contiguous())
    assert state.dtype == torch.float32 and state.shape[1:] == (k - 1, c)
    assert state.stride(2) == 1 and state.stride(1) == c
    _i32(cu, n_req + 1, "cu"); _i32(ctx, n_req, "ctx"); _i32(slot, n_req, "slot")
    if out is None:
        out = torch.empty((n_rows, c), dtype=bcx.dtype, device=bcx.device)
    assert out.shape == (n_rows, c) and out.dtype == bcx.dtype and out.is_contiguous()
    call("gibbs_shortconv", ptr(bcx), ptr(taps), ptr(bias), ptr(state), state.stride(0), ptr(cu), ptr(ctx),
         ptr(slot), ptr(out), dtype_code(bcx.dtype), n_rows, n_req,
         (n_req if n_rows == n_req else 0) if lead_single is None else int(lead_single), c, k, stream())
    return out


def _check_pages(pages: torch.Tensor, nkv: int, hd: int, dtype: torch.dtype) -> tuple[int, int]:
    assert pages.dim() == 4 and pages.shape[1] == nkv and pages.shape[3] == hd, (pages.shape, nkv, hd)
    assert pages.is_contiguous() and pages.dtype == dtype
    return pages.shape[0], pages.shape[2]


def qk_rope_kv(qkv: torch.Tensor, n_rows: int, nh: int, nkv: int, hd: int, *, q_gain: Optional[torch.Tensor],
               k_gain: Optional[torch.Tensor], eps: float, inv_freq: Optional[torch.Tensor], rotary_dim: int,
               variant: str, pos: torch.Tensor, row_req: torch.Tensor, kpages: Optional[torch.Tensor],
               vpages: Optional[torch.Tensor], table: Optional[torch.Tensor], n_req: int,
               cos_sin: Optional[torch.Tensor] = None) -> None:
    """In place on the q heads of qkv[N, (nh + 2 nkv) hd]: per-head RMSNorm then rotation; k heads the
    same and into their cache page; v heads copied to theirs.  With kpages None only q is treated
    (nkv then counts the k, v heads that the rows hold, usually 0).  `cos_sin`: what `rope_table`
    made for these frequencies; positions beyond it are computed in the kernel."""
    require_cuda(qkv, q_gain, k_gain, inv_freq, pos, row_req, kpages, vpages, table, cos_sin)
    table_len = _check_cos_sin(cos_sin, inv_freq, rotary_dim)
    assert qkv.dim() == 2 and qkv.shape[0] == n_rows and qkv.stride(1) == 1
    assert qkv.shape[1] >= (nh + 2 * nkv) * hd
    for g in (q_gain, k_gain):
        assert g is None or (g.dtype == torch.float32 and g.shape == (hd,) and g.is_contiguous())
    if inv_freq is not None:
        assert inv_freq.dtype == torch.float32 and inv_freq.shape == (rotary_dim // 2,) and inv_freq.is_contiguous()
    if variant not in ROPE_VARIANTS:
        raise KernelError(f"rotation variant {variant!r} is not implemented; known: {sorted(ROPE_VARIANTS)}")
    _i32(pos, n_rows, "pos"); _i32(row_req, n_rows, "row_req")
    num_pages = page_size = max_pages = 0
    if kpages is not None:
        num_pages, page_size = _check_pages(kpages, nkv, hd, qkv.dtype)
        assert _check_pages(vpages, nkv, hd, qkv.dtype) == (num_pages, page_size)
        assert table is not None and table.dim() == 2 and table.shape[0] >= n_req
        _i32(table, n_req, "block table")
        max_pages = table.shape[1]
    call("gibbs_qk_rope_kv", ptr(qkv), ptr(kpages), ptr(vpages), dtype_code(qkv.dtype), ptr(q_gain), ptr(k_gain),
         float(eps), ptr(inv_freq), rotary_dim, ROPE_VARIANTS[variant], ptr(cos_sin), table_len, ptr(pos),
         ptr(row_req), ptr(table), max_pages, page_size, num_pages, n_rows, nh, nkv, hd,
         qkv.stride(0) if n_rows > 1 else qkv.shape[1], stream())


def _check_cos_sin(cos_sin: Optional[torch.Tensor], inv_freq: Optional[torch.Tensor], rotary_dim: int) -> int:
    if cos_sin is None or inv_freq is None:
        return 0
    assert cos_sin.dtype == torch.float32 and cos_sin.dim() == 3 and cos_sin.is_contiguous()
    assert cos_sin.shape[1:] == (rotary_dim // 2, 2), "the cos/sin table belongs to another rotary size"
    return cos_sin.shape[0]


def rope_table(inv_freq: torch.Tensor, n_pos: int) -> torch.Tensor:
    """[n_pos, len(inv_freq), 2] float32: cos and sin of float32(pos) * inv_freq[j], computed by the
    functions that the kernels use for positions beyond a table."""
    require_cuda(inv_freq)
    assert inv_freq.dtype == torch.float32 and inv_freq.dim() == 1 and inv_freq.is_contiguous() and n_pos > 0
    out = torch.empty((n_pos, inv_freq.shape[0], 2), dtype=torch.float32, device=inv_freq.device)
    call("gibbs_rope_table", ptr(out), ptr(inv_freq), inv_freq.shape[0], n_pos, stream())
    return out


def attention_plain(q: torch.Tensor, n_rows: int, nh: int, nkv: int, hd: int, kpages: torch.Tensor,
                    vpages: torch.Tensor, table: torch.Tensor, n_req: int, pos: torch.Tensor, row_req: torch.Tensor,
                    scale: float, window: Optional[int] = None, out: Optional[torch.Tensor] = None,
                    slopes: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Causal grouped-query attention of every row over its request's cache pages.
    q: [N, >= nh*hd] (row stride free); pages: [num_pages, nkv, page_size, hd]; table: [R, max_pages].
    `slopes` (float32 [nh]): the score of key k for a query at position p gets slopes[h] * (k - p) added."""
    require_cuda(q, kpages, vpages, table, pos, row_req, slopes)
    assert slopes is None or (slopes.dtype == torch.float32 and slopes.shape == (nh,) and slopes.is_contiguous())
    assert q.dim() == 2 and q.shape[0] == n_rows and q.stride(1) == 1 and q.shape[1] >= nh * hd
    num_pages, page_size = _check_pages(kpages, nkv, hd, q.dtype)
    assert _check_pages(vpages, nkv, hd, q.dtype) == (num_pages, page_size)
    assert table.dim() == 2 and table.shape[0] >= n_req
    _i32(table, n_req, "block table"); _i32(pos, n_rows, "pos"); _i32(row_req, n_rows, "row_req")
    if out is None:
        out = torch.empty((n_rows, nh * hd), dtype=q.dtype, device=q.device)
    assert out.shape == (n_rows, nh * hd) and out.dtype == q.dtype and out.is_contiguous()
    call("gibbs_attention_plain", ptr(q), ptr(kpages), ptr(vpages), ptr(out), dtype_code(q.dtype), ptr(pos),
         ptr(row_req), ptr(table), table.shape[1], page_size, num_pages, n_rows, nh, nkv, hd,
         q.stride(0) if n_rows > 1 else q.shape[1], nh * hd, float(scale), int(window or 0), ptr(slopes), stream())
    return out


# how the decode attention walks its keys: chosen by the kernel, on the vector units, on the matrix cores
# (+ 4, "-merge-pass": the key slices are merged by a second kernel instead of by the slice that finishes last)
DECODE_KINDS = {"auto": 0, "valu": 1, "mfma": 2, "auto-merge-pass": 4, "valu-merge-pass": 5, "mfma-merge-pass": 6}


def slices_workspace(n_rows: int, nh: int, hd: int, n_splits: int) -> int:
    """Floats that the key slices of an attention call leave for the merge kernel."""
    return int(library().gibbs_attention_decode_workspace(n_rows, nh, hd, n_splits))


def decode_splits(n_rows: int, nkv: int, group: int, max_seq: int, hd: int = 0, kind: str = "auto",
                  page_size: int = 16) -> tuple:
    """(key slices per (row, kv head), waves per workgroup) that the native step would choose for the
    decode attention (csrc/step_plan.hip)."""
    import ctypes
    n_splits, waves = ctypes.c_int(0), ctypes.c_int(0)
    library().gibbs_rule_decode_splits(n_rows, nkv, group, max_seq, hd, page_size, DECODE_KINDS[kind], ctypes.byref(n_splits),
                                       ctypes.byref(waves))
    return n_splits.value, waves.value


def attention_decode(q: torch.Tensor, n_rows: int, nh: int, nkv: int, hd: int, kpages: torch.Tensor,
                     vpages: torch.Tensor, table: torch.Tensor, n_req: int, pos: torch.Tensor, row_req: Optional[torch.Tensor],
                     scale: float, window: Optional[int] = None, max_seq: int = 0, n_splits: Optional[int] = None,
                     out: Optional[torch.Tensor] = None, waves: Optional[int] = None, kind: str = "auto") -> torch.Tensor:
    """bfloat16 paged attention for rows with few queries and long caches (decoded tokens): the
    keys of each (row, kv head) are cut into `n_splits` slices that run as workgroups of their own
    and are merged afterwards.  Same operands and result as `attention_plain`; `row_req` None says that row n is
    request n.  `max_seq`, if given, bounds the keys of every row; it steers how the kernel asks for page ids and
    cuts slices (a row beyond it is still right as long as a slice's page ids fit the kernel's staging area)."""
    require_cuda(q, kpages, vpages, table, pos, row_req)
    if q.dtype != torch.bfloat16:
        raise KernelError("attention_decode is the bfloat16 kernel; the float32 path uses attention_plain")
    assert q.dim() == 2 and q.shape[0] == n_rows and q.stride(1) == 1 and q.shape[1] >= nh * hd
    if hd % 8 or hd > 256:
        raise KernelError(f"attention_decode: head size {hd} must be a multiple of 8 up to 256")
    num_pages, page_size = _check_pages(kpages, nkv, hd, q.dtype)
    assert _check_pages(vpages, nkv, hd, q.dtype) == (num_pages, page_size)
    assert table.dim() == 2 and table.shape[0] >= n_req
    _i32(table, n_req, "block table"); _i32(pos, n_rows, "pos")
    if row_req is not None:   # (None: row n is request n)
        _i32(row_req, n_rows, "row_req")
    else:
        assert n_rows <= table.shape[0], "rows without a row-to-request map are requests"
    if n_splits is None or waves is None:
        auto_splits, auto_waves = decode_splits(n_rows, nkv, nh // nkv, max_seq, hd, kind, page_size)
        n_splits = auto_splits if n_splits is None else n_splits
        waves = auto_waves if waves is None else waves
    partial = None
    if n_splits > 1:
        partial = torch.empty(slices_workspace(n_rows, nh, hd, n_splits), dtype=torch.float32, device=q.device)
    if out is None:
        out = torch.empty((n_rows, nh * hd), dtype=q.dtype, device=q.device)
    assert out.shape == (n_rows, nh * hd) and out.dtype == q.dtype and out.is_contiguous()
    call("gibbs_attention_decode", ptr(q), ptr(kpages), ptr(vpages), ptr(out), ptr(partial), ptr(pos), ptr(row_req),
         ptr(table), table.shape[1], page_size, num_pages, n_rows, nh, nkv, hd,
         q.stride(0) if n_rows > 1 else q.shape[1], nh * hd, float(scale), int(window or 0), n_splits, int(waves), DECODE_KINDS[kind], int(max_seq), stream())
    return out


def prefill_splits(n_tiles: int, nh: int, max_seq: int, window: Optional[int] = None) -> int:
    """Slices of the key tiles that the native step would choose for the prompt attention (csrc/step_plan.hip)."""
    return int(library().gibbs_rule_prefill_splits(n_tiles, nh, max_seq, int(window or 0)))


def attention_prefill(q: torch.Tensor, n_rows: int, nh: int, nkv: int, hd: int, kpages: torch.Tensor,
                      vpages: torch.Tensor, table: torch.Tensor, n_req: int, cu: torch.Tensor, ctx: torch.Tensor,
                      scale: float, window: Optional[int] = None, out: Optional[torch.Tensor] = None,
                      max_seq: int = 0, n_splits: Optional[int] = None, first_req: int = 0,
                      first_row: int = 0, heads_per_wg: Optional[int] = None) -> torch.Tensor:
    """bfloat16 paged causal attention for prompt portions on the matrix cores: rows cu[r] .. cu[r+1]
    of request r sit at positions ctx[r] ..; same result as `attention_plain`.  Head sizes: multiples
    of 16 up to 128.  `max_seq`: a bound on the keys of any row, from which the number of key slices
    is chosen (or `n_splits`).  `first_req`, `first_row`: only the requests from `first_req` on are
    attended to (their rows start at `first_row`); the rows before are left as they are in `out`.
    `heads_per_wg`: query heads of a kv head's group per workgroup (1, 2 or 4; default: the native step's rule)."""
    require_cuda(q, kpages, vpages, table, cu, ctx)
    if q.dtype != torch.bfloat16:
        raise KernelError("attention_prefill is the bfloat16 kernel; the float32 path uses attention_plain")
    if hd % 16 or not 16 <= hd <= 128:
        raise KernelError(f"attention_prefill: head size {hd} must be a multiple of 16 up to 128")
    assert q.dim() == 2 and q.shape[0] == n_rows and q.stride(1) == 1 and q.shape[1] >= nh * hd
    num_pages, page_size = _check_pages(kpages, nkv, hd, q.dtype)
    assert _check_pages(vpages, nkv, hd, q.dtype) == (num_pages, page_size)
    assert table.dim() == 2 and table.shape[0] >= n_req
    _i32(table, n_req, "block table"); _i32(cu, n_req + 1, "cu"); _i32(ctx, n_req, "ctx")
    assert 0 <= first_req <= n_req and 0 <= first_row <= n_rows
    if out is None:
        out = torch.empty((n_rows, nh * hd), dtype=q.dtype, device=q.device)
    assert out.shape == (n_rows, nh * hd) and out.dtype == q.dtype and out.is_contiguous()
    rows, reqs = n_rows - first_row, n_req - first_req
    if n_splits is None:
        n_splits = prefill_splits(int(library().gibbs_rule_prefill_tiles(rows, reqs)), nh, max_seq, window) if max_seq > 0 else 1
    if heads_per_wg is None:
        heads_per_wg = int(library().gibbs_rule_prefill_heads(rows, reqs, nh, nkv, hd, int(max_seq), int(n_splits)))
    partial = None
    if n_splits > 1:
        partial = torch.empty(slices_workspace(n_rows, nh, hd, n_splits), dtype=torch.float32, device=q.device)
    call("gibbs_attention_prefill", ptr(q), ptr(kpages), ptr(vpages), ptr(out), ptr(partial), ptr(cu[first_req:]),
         ptr(ctx[first_req:]), ptr(table[first_req:]), reqs, table.shape[1], page_size, num_pages, rows, nh, nkv, hd,
         q.stride(0) if n_rows > 1 else q.shape[1], nh * hd, float(scale), int(window or 0), int(n_splits), int(first_row),
         int(heads_per_wg), stream())
    return out


def probe_read(buffer: torch.Tensor, offset: int, nbytes: int, out: torch.Tensor, grid: int = 1024, block: int = 256) -> None:
    """Reads `nbytes` of `buffer` from byte `offset` and leaves per-workgroup sums in `out` (float32 [grid]): the
    yardstick for the weight-streaming kernels (measurement only)."""
    require_cuda(buffer, out)
    assert buffer.is_contiguous() and 0 <= offset and offset + nbytes <= buffer.numel() * buffer.element_size()
    assert out.dtype == torch.float32 and out.numel() >= grid and out.is_contiguous()
    call("gibbs_probe_read", buffer.data_ptr() + offset, nbytes, ptr(out), grid, block, stream())


def argmax(logits: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Index of the first largest value of each row (NaN never wins), int32 [M]."""
    require_cuda(logits)
    m, v = logits.shape
    assert logits.dtype == torch.float32 and logits.stride(1) == 1
    if out is None:
        out = torch.empty((m,), dtype=torch.int32, device=logits.device)
    _i32(out, m, "out")
    call("gibbs_argmax", ptr(logits), ptr(out), m, v, logits.stride(0) if m > 1 else v, stream())
    return out


def repetition_penalty(logits: torch.Tensor, recent: torch.Tensor, penalty: torch.Tensor,
                       temperature: torch.Tensor) -> torch.Tensor:
    """Penalises, in place, the logits of the tokens in `recent` [M, R] (int32, negative: none) by the
    reference's rule for greedy rows (temperature <= 1e-4) or sampled rows; rows with penalty <= 1
    are left alone."""
    require_cuda(logits, recent, penalty, temperature)
    m, v = logits.shape
    assert logits.dtype == torch.float32 and logits.stride(1) == 1
    assert recent.dtype == torch.int32 and recent.dim() == 2 and recent.shape[0] == m and recent.is_contiguous()
    for t in (penalty, temperature):
        assert t.dtype == torch.float32 and t.numel() >= m and t.is_contiguous()
    call("gibbs_repetition_penalty", ptr(logits), m, v, logits.stride(0) if m > 1 else v, ptr(recent), recent.shape[1],
         ptr(penalty), ptr(temperature), stream())
    return logits


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_p: torch.Tensor, top_k: torch.Tensor,
           u: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """One token per row: top-k, softmax at the row's temperature, top-p cut, draw with u in [0, 1)."""
    require_cuda(logits, temperature, top_p, top_k, u)
    m, v = logits.shape
    assert logits.dtype == torch.float32 and logits.stride(1) == 1
    for t in (temperature, top_p, u):
        assert t.dtype == torch.float32 and t.numel() >= m and t.is_contiguous()
    _i32(top_k, m, "top_k")
    if out is None:
        out = torch.empty((m,), dtype=torch.int32, device=logits.device)
    _i32(out, m, "out")
    call("gibbs_sample", ptr(logits), ptr(out), m, v, logits.stride(0) if m > 1 else v, ptr(temperature),
         ptr(top_p), ptr(top_k), ptr(u), stream())
    return out


def decode_tail(logits: Optional[torch.Tensor], ids: torch.Tensor, pos: torch.Tensor, ctx: torch.Tensor, log: torch.Tensor,
                steps: torch.Tensor, u: Optional[torch.Tensor], u_all: Optional[torch.Tensor], n: int,
                table: Optional[torch.Tensor] = None, x: Optional[torch.Tensor] = None,
                mirror: Optional[torch.Tensor] = None, live: Optional[torch.Tensor] = None) -> None:
    """End of a decode step on the device, one kernel: with `logits` the rows' next tokens are their first
    largest logits (else `ids` hold them already); the tokens are logged (log[steps[i], i]), pos and ctx move
    on by one, the next draws are loaded, steps[i] counts; with `table` and `x` the tokens' embeddings become
    the rows of the next step's residual stream x [n, hidden] (float32) and of its bfloat16 `mirror`.  `live`
    (int32 [n]): rows with 0 stand for no request: nothing of theirs is logged or moves on, they only get the
    embedding of the token they hold again."""
    require_cuda(logits, ids, pos, ctx, log, steps, u, u_all, table, x, mirror, live)
    if live is not None:
        _i32(live, n, "live")
    for t, what in ((pos, "pos"), (ctx, "ctx"), (ids, "ids"), (steps, "steps")):
        _i32(t, n, what)
    assert log.dtype == torch.int32 and log.is_contiguous() and log.numel() % n == 0
    capacity = log.numel() // n
    v = ld = 0
    if logits is not None:
        assert logits.dtype == torch.float32 and logits.dim() == 2 and logits.shape[0] == n and logits.stride(1) == 1
        v, ld = logits.shape[1], logits.stride(0) if n > 1 else logits.shape[1]
    if u is not None:
        assert u.dtype == torch.float32 and u.numel() >= n and u_all is not None
        assert u_all.dtype == torch.float32 and u_all.is_contiguous() and u_all.numel() >= capacity * n
    vocab = hidden = 0
    if x is not None:
        assert table is not None and table.dim() == 2 and table.is_contiguous()
        vocab, hidden = table.shape
        assert x.dtype == torch.float32 and x.shape == (n, hidden) and x.is_contiguous()
        assert mirror is None or (mirror.dtype == torch.bfloat16 and mirror.shape == (n, hidden) and mirror.is_contiguous())
    call("gibbs_decode_tail", ptr(logits), v, ld, ptr(ids), ptr(pos), ptr(ctx), ptr(log), ptr(steps), n, capacity, ptr(u),
         ptr(u_all), ptr(table), dtype_code(table.dtype) if table is not None else 0, vocab, hidden, ptr(x),
         ptr(mirror) if x is not None else None, ptr(live), stream())
