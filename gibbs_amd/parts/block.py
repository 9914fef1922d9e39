"""Arrangements of a layer's parts.

`pre_norm` is LFM2's (arch/families/lfm2.json5:77-88):
    x = x + mixer(norm(x));   x = x + ffn(norm(x))
The residual stream x is float32.  On the general path each residual add is fused into the norm
that follows it, so a block hands its last delta on instead of adding it.

In bfloat16 the block folds each norm's gain into the matrices that read the normed rows (the
reference's graph passes fold norm gains into weights too, src/graph/passes/mod.rs).
A step of single decoded tokens (up to `Runtime.fused_decode_rows` rows, at most 64) then takes the parts' fused decode kernels: the
product itself computes 1/rms of its input rows, and the last product of each half adds its result
into the stream, so a half of a layer is two or three kernels.
"""
from __future__ import annotations

import torch

from .. import ops
from .base import Block, Runtime, Stream, register_arrangement

# rows (decoded tokens) that the fused decode kernels take at most
MAX_FUSED_DECODE_ROWS = 64


def fused_decode_step(rt: Runtime, batch) -> bool:
    """Whether this step (every row one decoded token, few enough of them) may take the fused decode kernels."""
    return (rt.act_dtype == torch.bfloat16 and batch is not None and batch.max_q == 1
            and batch.n_rows <= min(rt.fused_decode_rows, MAX_FUSED_DECODE_ROWS))


@register_arrangement("pre_norm")
class PreNormBlock(Block):
    def bind(self, weights, rt: Runtime) -> None:
        super().bind(weights, rt)
        self.mixer_folded = self._fold(self.mixer_norm, self.mixer)
        self.ffn_folded = self._fold(self.ffn_norm, self.ffn)
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

    def _fused(self, part, folded: bool, batch, cache=None) -> bool:
        return (folded and fused_decode_step(self.rt, batch) and hasattr(part, "decode_fused")
                and part.can_decode_fused(batch))

    def emit_native(self, builder, cache) -> bool:
        """Lays the block down in the native step's plan; False if one of its parts cannot."""
        parts = (self.mixer_norm, self.ffn_norm, self.mixer, self.ffn)
        if not all(hasattr(p, "native_norm") for p in parts[:2]) or not all(hasattr(p, "emit_native") for p in parts[2:]):
            return False
        (g1, e1), (g2, e2) = self.mixer_norm.native_norm(), self.ffn_norm.native_norm()
        builder.block(g1, e1, g2, e2)
        return (self.mixer.emit_native(builder, cache, self.mixer_folded)
                and self.ffn.emit_native(builder, self.ffn_folded))

    def forward(self, stream: Stream, batch, cache) -> Stream:
        if self._fused(self.mixer, self.mixer_folded, batch):
            self.mixer.decode_fused(stream.with_mirror(), self.mixer_norm.spec.eps, batch, cache)
        else:
            stream.add(self.mixer.forward(stream.normed(self.mixer_norm), batch, cache))   # (the add waits for the next norm)
        if self._fused(self.ffn, self.ffn_folded, batch):
            self.ffn.decode_fused(stream.with_mirror(), self.ffn_norm.spec.eps, batch)
        else:
            stream.add(self.ffn.forward(stream.normed(self.ffn_norm), batch))
        return stream
