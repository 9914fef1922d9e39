"""Gated short-convolution mixer (the reference's `shortconv` block, arch/lib/transformer.json5:138-151).

[B | C | x] = thirds of in_proj(h), in that order; bx = B * x; a depthwise causal convolution of
length K over bx whose history is the request's state (the last K-1 rows of bx, oldest first,
zeros at a sequence start; src/graph/cpu.rs:952-994); y = C * conv; out_proj(y).
The reference refuses a convolution bias (arch/families/lfm2.json5:53); here
`bias: true` adds it after the tap sum.
"""
from __future__ import annotations

from typing import List, Sequence

import torch

from .. import ops
from ..cache.needs import StateNeed
from ..weights.loader import FLOAT32, TensorDecl, WeightStore
from .base import Mixer, Runtime, register_mixer

STATE = "conv"


@register_mixer("short_conv")
class ShortConvMixer(Mixer):
    def __init__(self, spec, hidden, layer_index):
        super().__init__(spec, hidden, layer_index)
        p = spec.params
        self.width, self.kernel, self.bias = int(p["width"]), int(p["kernel"]), bool(p.get("bias", False))
        if self.kernel < 2:
            raise ValueError(f"a short convolution needs a kernel of at least 2 taps, not {self.kernel}")

    def state_needs(self) -> Sequence[StateNeed]:
        return (StateNeed(STATE, (self.kernel - 1, self.width)),)

    def tensor_decls(self) -> List[TensorDecl]:
        t, C, K = self.spec.tensors, self.width, self.kernel
        decls = [TensorDecl(t["in_proj"], (3 * C, self.hidden)),
                 # stored [width, 1, kernel]; [width, kernel] is the same data (lfm2.json5:58-62)
                 TensorDecl(t["conv"], (C, 1, K), FLOAT32, alt_shapes=((C, K),)),
                 TensorDecl(t["out_proj"], (self.hidden, C))]
        if self.bias:
            decls.append(TensorDecl(t["conv_bias"], (C,), FLOAT32, init="bias"))
        return decls

    def bind(self, weights: WeightStore, rt: Runtime) -> None:
        self.rt = rt
        t = self.spec.tensors
        self.w_in = weights[t["in_proj"]]
        self.taps = weights[t["conv"]].reshape(self.width, self.kernel).contiguous()
        self.w_out = weights[t["out_proj"]]
        self.p_in = self.p_out = None
        self.conv_bias = weights[t["conv_bias"]] if self.bias else None

    def matrices(self):
        return [self.w_in, self.w_out]

    def product_shapes(self):
        return [(3 * self.width, self.hidden), (self.hidden, self.width)]

    def small_tensors(self):
        return [self.taps] + ([self.conv_bias] if self.bias else [])

    def fold_input_gain(self, gain: torch.Tensor) -> None:
        """The preceding norm's gain, multiplied into the columns of the in-projection."""
        self.w_in = (self.w_in.float() * gain[None, :]).to(self.w_in.dtype)

    def pack_matrices(self) -> None:
        self.p_in = ops.PackedWeight(self.w_in, groups=3)
        self.p_out = ops.PackedWeight(self.w_out)

    def emit(self, plan, cache) -> int:
        return plan.short_conv(w_in=self.w_in, p_in=self.p_in, w_out=self.w_out, p_out=self.p_out, taps=self.taps,
                               bias=self.conv_bias, width=self.width, kernel=self.kernel, state=cache.states[STATE])
