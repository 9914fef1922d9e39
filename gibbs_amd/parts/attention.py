"""Grouped-query attention mixer over the paged cache.

In the reference's order (arch/lib/transformer.json5:46-87): q, k, v
projections; optional RMSNorm of every head of q and k with one [head_dim] gain (`qk_norm:
"before"` the rotation, as LFM2 has it, arch/families/lfm2.json5:80-83);
position encoding of q and k; k, v written to the cache at their positions; causal attention of
each row over the keys up to its own position (within `window`, if given), query head h reading
kv head h // (heads / kv_heads) with scale `scale`; output projection.  A mixer whose params
name `kv_source` projects no k, v and reads that layer's pages (the reference's `write: false`).

The position encoding is asked how it works (`PositionEncoding`): a rotation goes to the kernels
as tables and every fast path stays open; an encoding that changes q and k itself (`apply`) or
biases the scores by distance (`score_slopes`) sends the mixer down its general path (norm, the
hook, cache write; the plain attention kernel takes the slopes).
"""
from __future__ import annotations

from typing import List, Optional

import torch

from .. import ops
from ..cache.needs import CacheNeed
from ..ops.linear import linear
from ..weights.loader import FLOAT32, TensorDecl, WeightStore
from .base import Mixer, Runtime, build_position, register_mixer


MIN_LEADING_DECODED = 2      # decoded tokens at the head of a mixed step that are worth a kernel of their own


@register_mixer("attention")
class AttentionMixer(Mixer):
    def __init__(self, spec, hidden, layer_index):
        super().__init__(spec, hidden, layer_index)
        p = spec.params
        self.heads, self.kv_heads, self.head_dim = int(p["heads"]), int(p["kv_heads"]), int(p["head_dim"])
        self.scale = float(p["scale"])
        self.window = p.get("window")
        self.qk_norm = p.get("qk_norm")
        self.qk_norm_eps = float(p.get("qk_norm_eps", 0.0))
        self.source = p.get("kv_source")
        if self.heads % self.kv_heads:
            raise ValueError(f"{self.heads} heads are not a multiple of {self.kv_heads} kv heads")
        if self.qk_norm not in (None, "before"):
            raise ValueError(f"qk_norm {self.qk_norm!r} is not implemented (None or 'before')")
        if self.window is not None and int(self.window) <= 0:
            raise ValueError(f"attention window {self.window} must be positive")
        self.position = build_position(spec.position, self.head_dim)

    # ------------------------------------------------------------------ what it asks for
    def cache_need(self) -> Optional[CacheNeed]:
        if self.source is not None:
            return None
        return CacheNeed(self.kv_heads, self.head_dim, None if self.window is None else int(self.window))

    def attention_flops(self, keys: float) -> float:
        """Multiply-adds x 2 of scores and weighted values when the step's rows see `keys` keys in all."""
        return 2.0 * 2.0 * keys * self.heads * self.head_dim

    def kv_source(self) -> Optional[int]:
        return self.source

    def tensor_decls(self) -> List[TensorDecl]:
        t, H, hd = self.spec.tensors, self.hidden, self.head_dim
        decls = [TensorDecl(t["q_proj"], (self.heads * hd, H))]
        if self.source is None:
            decls += [TensorDecl(t["k_proj"], (self.kv_heads * hd, H)), TensorDecl(t["v_proj"], (self.kv_heads * hd, H))]
        decls.append(TensorDecl(t["out_proj"], (H, self.heads * hd)))
        if self.qk_norm:
            decls.append(TensorDecl(t["q_norm"], (hd,), FLOAT32, init="gain"))
            if self.source is None:
                decls.append(TensorDecl(t["k_norm"], (hd,), FLOAT32, init="gain"))
        if self.position is not None:
            decls += self.position.tensor_decls()
        return decls

    def bind(self, weights: WeightStore, rt: Runtime) -> None:
        self.rt = rt
        t = self.spec.tensors
        if self.source is None:
            # one product for q, k and v: rows [Wq; Wk; Wv]
            self.w_qkv = torch.cat([weights[t["q_proj"]], weights[t["k_proj"]], weights[t["v_proj"]]], dim=0).contiguous()
        else:
            self.w_qkv = weights[t["q_proj"]]
        self.w_out = weights[t["out_proj"]]
        self.p_qkv = self.p_out = None
        self.q_gain = weights[t["q_norm"]] if self.qk_norm else None
        self.k_gain = weights[t["k_norm"]] if self.qk_norm and self.source is None else None
        self.rot, self.slopes, self.pos_hook = None, None, False
        if self.position is not None:
            self.position.bind(weights, rt)
            self.rot = self.position.rotation()
            self.slopes = self.position.score_slopes(self.heads)
            self.pos_hook = self.rot is None and self.position.transforms_rows()
        if self.slopes is not None and (self.slopes.dtype != torch.float32 or tuple(self.slopes.shape) != (self.heads,)):
            raise ValueError(f"score slopes must be float32 [{self.heads}]")
        # the fast kernels know rotations only (or no encoding at all)
        self.fast_ok = self.slopes is None and not self.pos_hook

    def matrices(self):
        return [self.w_qkv, self.w_out]

    def product_shapes(self):
        kv = 2 * self.kv_heads if self.source is None else 0
        return [((self.heads + kv) * self.head_dim, self.hidden), (self.hidden, self.heads * self.head_dim)]

    def small_tensors(self):
        own = [t for t in (self.q_gain, self.k_gain, self.slopes) if t is not None]
        return own + ([] if self.position is None else list(self.position.small_tensors()))

    def fold_input_gain(self, gain: torch.Tensor) -> None:
        """The preceding norm's gain, multiplied into the columns of the q, k, v projections."""
        self.w_qkv = (self.w_qkv.float() * gain[None, :]).to(self.w_qkv.dtype)

    def pack_matrices(self) -> None:
        self.p_qkv = ops.PackedWeight(self.w_qkv)
        self.p_out = ops.PackedWeight(self.w_out)

    def _rotation_args(self) -> dict:
        """The rotation as the kernels take it (no rotation: nulls)."""
        r = self.rot
        if r is None:
            return dict(inv_freq=None, rotary_dim=0, variant="half_split", cos_sin=None)
        return dict(inv_freq=r.inv_freq, rotary_dim=r.rotary_dim, variant=r.variant, cos_sin=r.cos_sin)

    def can_decode_fused(self, batch) -> bool:
        rot_ok = self.fast_ok and (self.rot is None or self.rot.rotary_dim % 16 == 0)
        return (self.source is None and self.hidden % 8 == 0 and self.head_dim % 16 == 0 and self.head_dim <= 256
                and rot_ok and (self.heads * self.head_dim) % 8 == 0)

    def decode_fused(self, stream, norm_eps: float, batch, cache) -> None:
        """norm -> q, k, v in one kernel; q/k norm, rotation, the write of the new key and value and
        attention over split keys in a second (and the merge of the slices); out_proj + residual
        add in a third."""
        qkv = ops.skinny_store(stream.mirror, self.p_qkv or self.w_qkv, rms_eps=norm_eps)
        ops.skinny_residual(self._attend_decoded(qkv, batch, cache), self.p_out or self.w_out, stream.x, stream.mirror)

    def _attend_decoded(self, qkv, batch, cache) -> torch.Tensor:
        """A step of single decoded tokens, from the raw projection: one kernel norms and rotates q and
        the new key, writes key and value to their pages and attends."""
        return ops.attention_decode_fused(
            qkv, batch.n_rows, self.heads, self.kv_heads, self.head_dim, cache.kpages, cache.vpages,
            batch.tables[cache.group], batch.n_req, batch.pos, batch.row_req, self.scale, q_gain=self.q_gain,
            k_gain=self.k_gain, eps=self.qk_norm_eps, window=self.window, max_seq=batch.max_seq,
            **self._rotation_args())

    def emit_native(self, builder, cache, folded: bool) -> bool:
        if not self.fast_ok or cache.kpages is None or cache.kpages.shape != cache.vpages.shape:
            return False                # (an encoding with a hook or score slopes steps through `forward`)
        builder.attention(w_qkv=self.w_qkv, p_qkv=self.p_qkv, w_out=self.w_out, p_out=self.p_out, heads=self.heads,
                          kv_heads=self.kv_heads, head_dim=self.head_dim, scale=self.scale, window=self.window,
                          q_gain=self.q_gain, k_gain=self.k_gain, qk_eps=self.qk_norm_eps, rotation=self.rot,
                          kpages=cache.kpages, vpages=cache.vpages, group=cache.group, owns=self.source is None,
                          fusable=folded and self.can_decode_fused(None))
        return True

    # ------------------------------------------------------------------ one step
    def forward(self, h: torch.Tensor, batch, cache) -> torch.Tensor:
        n = batch.n_rows
        qkv = linear(h, self.w_qkv)
        table = batch.tables[cache.group]
        owns = self.source is None
        rot_ok = self.fast_ok and (self.rot is None or self.rot.rotary_dim % 16 == 0)
        if (owns and self.rt.act_dtype == torch.bfloat16 and batch.max_q == 1 and self.head_dim % 16 == 0
                and self.head_dim <= 256 and rot_ok):
            return linear(self._attend_decoded(qkv, batch, cache), self.w_out, partial_ok=True, packed=self.p_out)
        nkv = self.kv_heads if owns else 0
        where = dict(pos=batch.pos, row_req=batch.row_req, table=table, n_req=batch.n_req)
        pages = dict(kpages=cache.kpages if owns else None, vpages=cache.vpages if owns else None)
        if self.pos_hook:
            # q/k norm, then the encoding's own doing on the rows, then k and v into their pages
            hd = self.head_dim
            plain = dict(k_gain=None, eps=self.qk_norm_eps, **self._rotation_args(), **where)
            k_rows = qkv[:, self.heads * hd:(self.heads + nkv) * hd]
            if self.q_gain is not None:          # the kernel norms heads in place when it is given no pages
                ops.qk_rope_kv(qkv, n, self.heads, 0, hd, q_gain=self.q_gain, kpages=None, vpages=None, **plain)
            if owns and self.k_gain is not None:
                ops.qk_rope_kv(k_rows, n, nkv, 0, hd, q_gain=self.k_gain, kpages=None, vpages=None, **plain)
            self.position.apply(qkv[:, :self.heads * hd].unflatten(1, (self.heads, hd)),
                                k_rows.unflatten(1, (nkv, hd)) if owns else None, batch)
            if owns:
                ops.qk_rope_kv(qkv, n, self.heads, nkv, hd, q_gain=None, **pages, **plain)
        else:
            ops.qk_rope_kv(qkv, n, self.heads, nkv, self.head_dim, q_gain=self.q_gain, k_gain=self.k_gain,
                           eps=self.qk_norm_eps, **self._rotation_args(), **pages, **where)
        a = self.attend(qkv, batch, cache, table)
        return linear(a, self.w_out, partial_ok=True, packed=self.p_out)

    def attend(self, qkv, batch, cache, table) -> torch.Tensor:
        """Attention of the step's rows over the cache.  bfloat16: rows that are all single decoded
        tokens take the kernel that splits the keys, steps with prompt portions the matrix-core
        kernel (head sizes up to 128).  float32, and whatever the fast kernels do not take: the
        plain kernel."""
        bf16 = self.rt.act_dtype == torch.bfloat16 and self.slopes is None   # (the fast kernels take no score bias)
        if bf16 and batch.max_q > 1 and self.head_dim % 16 == 0 and self.head_dim <= 128:
            # decoded tokens at the head of the batch (where the scheduler puts them) take the kernel that
            # splits their keys; a row of its own in the matrix-core kernel would walk its cache alone
            lead = batch.lead_single if batch.lead_single >= MIN_LEADING_DECODED else 0
            out = torch.empty((batch.n_rows, self.heads * self.head_dim), dtype=qkv.dtype, device=qkv.device)
            if lead:
                ops.attention_decode(qkv[:lead], lead, self.heads, self.kv_heads, self.head_dim, cache.kpages,
                                     cache.vpages, table, batch.n_req, batch.pos[:lead], batch.row_req[:lead],
                                     self.scale, self.window, max_seq=batch.max_seq, out=out[:lead])
            return ops.attention_prefill(qkv, batch.n_rows, self.heads, self.kv_heads, self.head_dim, cache.kpages,
                                         cache.vpages, table, batch.n_req, batch.cu, batch.ctx, self.scale, self.window,
                                         out=out, max_seq=batch.max_seq, first_req=lead, first_row=lead)
        if bf16 and batch.max_q == 1 and self.head_dim % 8 == 0:
            return ops.attention_decode(qkv, batch.n_rows, self.heads, self.kv_heads, self.head_dim, cache.kpages,
                                        cache.vpages, table, batch.n_req, batch.pos, batch.row_req, self.scale,
                                        self.window, max_seq=batch.max_seq)
        return ops.attention_plain(qkv, batch.n_rows, self.heads, self.kv_heads, self.head_dim, cache.kpages,
                                   cache.vpages, table, batch.n_req, batch.pos, batch.row_req, self.scale,
                                   self.window, slopes=self.slopes)
