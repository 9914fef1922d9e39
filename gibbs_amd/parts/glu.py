"""Dense gated feed-forward: down(act(gate(h)) * up(h)), `activation` one of `ops.ACTIVATIONS`; with "silu" this is
SwiGLU (arch/lib/transformer.json5:117-130, src/graph/cpu.rs:378-390).
Gate and up are one product against [W_gate; W_up]."""
from __future__ import annotations

from typing import List

import torch

from .. import ops
from ..weights.loader import TensorDecl, WeightStore
from .base import FeedForward, Runtime, register_feed_forward


@register_feed_forward("glu")
class GluFeedForward(FeedForward):
    def __init__(self, spec, hidden):
        super().__init__(spec, hidden)
        self.inter = int(spec.params["inter"])
        self.activation = spec.params.get("activation", "silu")
        if self.activation not in ops.ACTIVATIONS:
            raise ValueError(f"feed-forward activation {self.activation!r} is not implemented")

    def tensor_decls(self) -> List[TensorDecl]:
        t = self.spec.tensors
        return [TensorDecl(t["gate"], (self.inter, self.hidden)), TensorDecl(t["up"], (self.inter, self.hidden)),
                TensorDecl(t["down"], (self.hidden, self.inter))]

    def bind(self, weights: WeightStore, rt: Runtime) -> None:
        self.rt = rt
        t = self.spec.tensors
        self.w_gate_up = torch.cat([weights[t["gate"]], weights[t["up"]]], dim=0).contiguous()
        self.w_down = weights[t["down"]]
        self.p_gate_up = self.p_down = None

    def matrices(self):
        return [self.w_gate_up, self.w_down]

    def product_shapes(self):
        return [(2 * self.inter, self.hidden), (self.hidden, self.inter)]

    def fold_input_gain(self, gain: torch.Tensor) -> None:
        """The preceding norm's gain, multiplied into the columns of the gate and up matrices."""
        self.w_gate_up = (self.w_gate_up.float() * gain[None, :]).to(self.w_gate_up.dtype)

    def pack_matrices(self) -> None:
        self.p_gate_up = ops.PackedWeight(self.w_gate_up, groups=2)
        self.p_down = ops.PackedWeight(self.w_down)

    def emit(self, plan) -> int:
        return plan.glu(w_gate_up=self.w_gate_up, p_gate_up=self.p_gate_up, w_down=self.w_down, p_down=self.p_down,
                        inter=self.inter, activation=ops.ACTIVATIONS[self.activation])
