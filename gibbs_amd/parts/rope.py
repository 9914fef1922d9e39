"""Rotary position encoding: the table of inverse frequencies and the pairing variant that an
attention mixer hands to its kernel.

inv_freq[j] = 1 / theta^(2j / rotary_dim); with `precision: "f32"` every step of that is a
float32 operation, as LFM2's spec asks (src/arch/gen.rs:154-164,
arch/families/lfm2.json5:64).  The angle of position p is float32(p) * inv_freq[j]
(src/graph/cpu.rs:673); variant `half_split` turns the pair (j, j + rot/2),
`interleaved` the pair (2j, 2j + 1) (:676-695).

Cosine and sine of every angle up to the run's longest position are computed once, when the part is
bound, into a table that the kernels read (the same float32 angle, the same functions: positions
beyond the table are computed in the kernels and agree to the bit).
"""
from __future__ import annotations

import numpy as np
import torch

from .. import ops
from ..weights.loader import WeightStore
from .base import PositionEncoding, Rotation, Runtime, register_position


MAX_TABLE_POSITIONS = 1 << 20   # 8 bytes * rotary_dim / 2 each


def rope_inv_freq(rotary_dim: int, theta: float, precision: str = "f64") -> np.ndarray:
    half = rotary_dim // 2
    if precision == "f32":
        t = np.float32(theta)
        return np.array([np.float32(1.0) / np.power(t, np.float32(2 * j) / np.float32(rotary_dim), dtype=np.float32)
                         for j in range(half)], dtype=np.float32)
    if precision == "f64":
        return np.array([1.0 / (float(theta) ** (2.0 * j / rotary_dim)) for j in range(half)]).astype(np.float32)
    raise ValueError(f"rope precision {precision!r} is neither 'f32' nor 'f64'")


@register_position("rope")
class RotaryPosition(PositionEncoding):
    def __init__(self, spec, head_dim):
        super().__init__(spec, head_dim)
        p = spec.params
        self.rotary_dim = int(p.get("rotary_dim", head_dim))
        self.variant = p.get("variant", "half_split")
        self.theta = float(p["theta"])
        self.precision = p.get("precision", "f64")
        if self.rotary_dim <= 0 or self.rotary_dim % 2 or self.rotary_dim > head_dim:
            raise ValueError(f"rotary_dim {self.rotary_dim} must be even and within the head size {head_dim}")
        if self.variant not in ("half_split", "interleaved"):
            raise ValueError(f"rope variant {self.variant!r} is not implemented")

    def bind(self, weights: WeightStore, rt: Runtime) -> None:
        self.rt = rt
        n_pos = min(int(rt.max_positions), MAX_TABLE_POSITIONS)
        key = ("rope", self.rotary_dim, self.theta, self.precision, n_pos)
        if key not in rt.shared:        # the layers of a model that have the same encoding share one table
            inv_freq = torch.from_numpy(rope_inv_freq(self.rotary_dim, self.theta, self.precision)).to(rt.device)
            rt.shared[key] = (inv_freq, ops.rope_table(inv_freq, n_pos) if n_pos > 0 else None)
        self.inv_freq, self.cos_sin = rt.shared[key]

    def rotation(self) -> Rotation:
        return Rotation(self.inv_freq, self.rotary_dim, self.variant, self.cos_sin)

    def small_tensors(self):
        return [self.inv_freq]      # of the cos/sin table a step reads one row per token: not counted
