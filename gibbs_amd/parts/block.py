"""Arrangements of a layer's parts.

`pre_norm` is LFM2's (/root/reference/arch/families/lfm2.json5:77-88):
    x = x + mixer(norm(x));   x = x + ffn(norm(x))
The residual stream x is float32.  Each residual add is fused into the norm that follows it, so
a block hands its last delta on to the next block's (or the tail's) norm instead of adding it.
"""
from __future__ import annotations

from typing import Optional

import torch

from .base import Block, register_arrangement


@register_arrangement("pre_norm")
class PreNormBlock(Block):
    def forward(self, x: torch.Tensor, pending: Optional[torch.Tensor], batch, cache) -> torch.Tensor:
        h = self.mixer_norm.forward(x, pending)           # x += pending; h = norm(x)
        a = self.mixer.forward(h, batch, cache)
        h = self.ffn_norm.forward(x, a)                   # x += a; h = norm(x)
        return self.ffn.forward(h, batch)
