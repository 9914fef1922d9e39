"""Grouped-query attention mixer over the paged cache.

In the reference's order (arch/lib/transformer.json5:46-87): q, k, v
projections; optional RMSNorm of every head of q and k with one [head_dim] gain (`qk_norm:
"before"` the rotation, as LFM2 has it, arch/families/lfm2.json5:80-83);
position encoding of q and k; k, v written to the cache at their positions; causal attention of
each row over the keys up to its own position (within `window`, if given), query head h reading
kv head h // (heads / kv_heads) with scale `scale`; output projection.  A mixer whose params
name `kv_source` projects no k, v and reads that layer's pages (the reference's `write: false`).

The position encoding is asked how it works (`PositionEncoding`): a rotation goes to the kernels
as tables and every fast path stays open; an encoding that changes q and k itself (`apply`) is
called back between the q/k norm and the cache write, and one that biases the scores by distance
(`score_slopes`) takes the plain attention kernel, which knows such a bias.  Which kernels a step
takes is decided where the step runs (csrc/step_plan.hip).
"""
from __future__ import annotations

from typing import List, Optional

import torch

from .. import ops
from ..cache.needs import CacheNeed
from ..weights.loader import FLOAT32, TensorDecl, WeightStore
from .base import Mixer, Runtime, build_position, register_mixer


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

    def emit(self, plan, cache) -> int:
        if cache.kpages is None or cache.kpages.shape != cache.vpages.shape:
            raise ValueError("the attention mixer's kernels want keys and values of one head size")
        hook = self.position.apply if self.pos_hook else None
        return plan.attention(w_qkv=self.w_qkv, p_qkv=self.p_qkv, w_out=self.w_out, p_out=self.p_out, heads=self.heads,
                              kv_heads=self.kv_heads, head_dim=self.head_dim, scale=self.scale, window=self.window,
                              q_gain=self.q_gain, k_gain=self.k_gain, qk_eps=self.qk_norm_eps, rotation=self.rot,
                              kpages=cache.kpages, vpages=cache.vpages, group=cache.group, owns=self.source is None,
                              slopes=self.slopes, rows_hook=hook)
