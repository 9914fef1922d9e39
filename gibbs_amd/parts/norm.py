"""RMSNorm: out = x * 1/sqrt(mean(x^2) + eps) * gain, eps inside the root, the gain multiplied
last, no (1 + gain) offset (src/model/simd.rs:75-110,
arch/lib/transformer.json5:9-11)."""
from __future__ import annotations

from typing import List, Optional

import torch

from ..weights.loader import FLOAT32, TensorDecl, WeightStore
from .base import Norm, Runtime, register_norm


@register_norm("rms")
class RMSNorm(Norm):
    def tensor_decls(self) -> List[TensorDecl]:
        return [TensorDecl(self.spec.weight, (self.width,), FLOAT32, init="gain")]

    def bind(self, weights: WeightStore, rt: Runtime) -> None:
        self.rt = rt
        self.gain = weights[self.spec.weight]

    def fold_gain(self) -> torch.Tensor:
        """Hands the gain over to whoever multiplies it into the matrices that read the normed
        rows; from then on this norm only divides by the root mean square."""
        gain, self.gain = self.gain, None
        return gain

    def small_tensors(self):
        return [] if self.gain is None else [self.gain]

    def emit(self, plan) -> int:
        return plan.rms_norm(self.gain, self.spec.eps)
