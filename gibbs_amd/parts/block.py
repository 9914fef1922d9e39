"""Arrangements of a layer's parts.

`pre_norm` is LFM2's (arch/families/lfm2.json5:77-88):
    x = x + mixer(norm(x));   x = x + ffn(norm(x))
The residual stream x is float32.  In the native step each residual add is fused into the norm that
follows it, so a half of the block hands its delta on instead of adding it.

In bfloat16 the block folds each norm's gain into the matrices that read the normed rows (the
reference's graph passes fold norm gains into weights too, src/graph/passes/mod.rs).
A step of single decoded tokens (up to `Runtime.fused_decode_rows` rows) then takes the parts' fused
decode kernels: the product itself computes 1/rms of its input rows, and the last product of each
half adds its result into the stream, so a half of a layer is two or three kernels.  Whether a step
does is decided where the step runs (csrc/step_plan.hip), per half, from the step's shape, the
norm (its gain folded) and the part (sizes that its fused kernels take).
"""
from __future__ import annotations

import torch

from .base import Block, Runtime, register_arrangement


@register_arrangement("pre_norm")
class PreNormBlock(Block):
    def __init__(self, spec, hidden, layer_index):
        super().__init__(spec, hidden, layer_index)
        missing = [r for r in spec.PRE_NORM_ROLES if r not in self.named]
        if missing:
            raise ValueError(f"a pre-norm block needs the parts {list(spec.PRE_NORM_ROLES)}; layer {spec.name!r} lacks {missing}")

    def bind(self, weights, rt: Runtime) -> None:
        super().bind(weights, rt)
        self._fold(self.mixer_norm, self.mixer)
        self._fold(self.ffn_norm, self.ffn)
        if self.rt.act_dtype == torch.bfloat16:
            self.mixer.pack_matrices()
            self.ffn.pack_matrices()

    def _fold(self, norm, part) -> bool:
        if self.rt.act_dtype != torch.bfloat16 or not self.rt.fold_gains:
            return False
        if not (hasattr(norm, "fold_gain") and hasattr(part, "fold_input_gain")):
            return False
        part.fold_input_gain(norm.fold_gain())
        return True

    def emit(self, plan, caches) -> None:
        plan.half(self.mixer_norm.emit(plan), self.mixer.emit(plan, caches["mixer"]))
        plan.half(self.ffn_norm.emit(plan), self.ffn.emit(plan))
