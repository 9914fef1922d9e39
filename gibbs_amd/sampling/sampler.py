"""Greedy and temperature sampling on the device, with the reference's pipeline and defaults:
temperature <= 1e-4 is the first maximum; else top-k (50, at most 64) by (logit descending, id
ascending), softmax at the temperature, the shortest prefix reaching top_p, and a draw
(/root/reference/src/runtime/lm.rs:1043-1240, /root/reference/src/scheduler/mod.rs:171-178,
:335-339)."""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Sequence

import numpy as np
import torch

from .. import ops
from .rng import request_key, uniform

DEFAULT_MAX_NEW_TOKENS = 64        # scheduler/mod.rs:335
DEFAULT_TEMPERATURE = 1.0          # scheduler/mod.rs:337
DEFAULT_TOP_P = 0.9                # scheduler/mod.rs:339
DEFAULT_TOP_K = 50                 # scheduler/mod.rs:178
MAX_TOP_K = 64                     # runtime/lm.rs:1161
GREEDY_BELOW = 1e-4                # runtime/lm.rs:1073


@dataclass(frozen=True)
class SamplingParams:
    """Per-request sampling controls; None takes the default (scheduler/mod.rs:407-434)."""
    temperature: Optional[float] = None
    top_p: Optional[float] = None
    top_k: int = DEFAULT_TOP_K
    max_new_tokens: int = DEFAULT_MAX_NEW_TOKENS
    seed: int = 0
    ignore_eos: bool = False

    def __post_init__(self):
        if not 1 <= self.top_k <= MAX_TOP_K:
            raise ValueError(f"top_k ({self.top_k}) must be in 1..{MAX_TOP_K}")
        if self.max_new_tokens < 0:
            raise ValueError("max_new_tokens must not be negative")

    @property
    def resolved_temperature(self) -> float:
        return DEFAULT_TEMPERATURE if self.temperature is None else float(self.temperature)

    @property
    def resolved_top_p(self) -> float:
        return DEFAULT_TOP_P if self.top_p is None else float(self.top_p)

    @property
    def greedy(self) -> bool:
        return self.resolved_temperature <= GREEDY_BELOW


@dataclass(frozen=True)
class Draw:
    """What one row's sample depends on: its request's parameters, identity and output index."""
    params: SamplingParams
    rid: object
    index: int


class Sampler:
    def __init__(self, device: torch.device):
        self.device = device

    def sample(self, logits: torch.Tensor, draws: Sequence[Draw]) -> List[int]:
        """One token id per row of float32 logits [M, V]."""
        m = logits.shape[0]
        assert m == len(draws)
        if m == 0:
            return []
        if all(d.params.greedy for d in draws):
            return ops.argmax(logits).tolist()
        host = np.empty((4, m), dtype=np.float32)
        for i, d in enumerate(draws):
            host[0, i] = d.params.resolved_temperature
            host[1, i] = d.params.resolved_top_p
            host[2, i] = uniform(d.params.seed, request_key(d.rid), d.index)
        host[3].view(np.int32)[:] = [d.params.top_k for d in draws]
        dev = torch.from_numpy(host).to(self.device)
        return ops.sample(logits, dev[0], dev[1], dev[3].view(torch.int32), dev[2]).tolist()
