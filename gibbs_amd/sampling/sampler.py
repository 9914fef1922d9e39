"""Greedy and temperature sampling on the device, with the reference's pipeline and defaults:
temperature <= 1e-4 is the first maximum; else top-k (50, at most 64) by (logit descending, id
ascending), softmax at the temperature, the shortest prefix reaching top_p, and a draw
(src/runtime/lm.rs:1043-1240, src/scheduler/mod.rs:171-178,
:335-339).  The reference's sampler also takes a repetition penalty over the last 64 tokens
(lm.rs:1084-1105, :1163-1189), which its scheduler leaves at 1.0 (scheduler/mod.rs:178); here it is
a per-request parameter with the same default."""
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
RECENT_TOKENS = 64                 # the window the sampler sees (scheduler/mod.rs:33-36)


@dataclass(frozen=True)
class SamplingParams:
    """Per-request sampling controls; None takes the default (scheduler/mod.rs:407-434)."""
    temperature: Optional[float] = None
    top_p: Optional[float] = None
    top_k: int = DEFAULT_TOP_K
    max_new_tokens: int = DEFAULT_MAX_NEW_TOKENS
    seed: int = 0
    ignore_eos: bool = False
    repetition_penalty: float = 1.0     # > 1 penalises the tokens among the last 64 (off in the reference's scheduler)

    def __post_init__(self):
        if not 1 <= self.top_k <= MAX_TOP_K:
            raise ValueError(f"top_k ({self.top_k}) must be in 1..{MAX_TOP_K}")
        if self.max_new_tokens < 0:
            raise ValueError("max_new_tokens must not be negative")
        if not self.repetition_penalty > 0:
            raise ValueError("repetition_penalty must be positive (1.0: none)")

    @property
    def resolved_temperature(self) -> float:
        return DEFAULT_TEMPERATURE if self.temperature is None else float(self.temperature)

    @property
    def resolved_top_p(self) -> float:
        return DEFAULT_TOP_P if self.top_p is None else float(self.top_p)

    @property
    def greedy(self) -> bool:
        return self.resolved_temperature <= GREEDY_BELOW

    @property
    def penalises(self) -> bool:
        return self.repetition_penalty > 1.0


@dataclass(frozen=True)
class Draw:
    """What one row's sample depends on: its request's parameters, identity and output index, and
    (for a repetition penalty) the request's last tokens, prompt and output alike."""
    params: SamplingParams
    rid: object
    index: int
    recent: Sequence[int] = ()


class Sampler:
    def __init__(self, device: torch.device):
        self.device = device

    def sample(self, logits: torch.Tensor, draws: Sequence[Draw]) -> List[int]:
        """One token id per row of float32 logits [M, V]."""
        m = logits.shape[0]
        assert m == len(draws)
        if m == 0:
            return []
        if any(d.params.penalises and len(d.recent) for d in draws):
            logits = self._penalised(logits, draws)
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

    def _penalised(self, logits: torch.Tensor, draws: Sequence[Draw]) -> torch.Tensor:
        """A copy of the logits with the repetition penalty of every row that asks for one."""
        m = logits.shape[0]
        host = np.full((m, RECENT_TOKENS + 2), -1, dtype=np.int32)
        floats = host[:, RECENT_TOKENS:].view(np.float32)
        for i, d in enumerate(draws):
            recent = list(d.recent)[-RECENT_TOKENS:] if d.params.penalises else []
            host[i, :len(recent)] = recent
            floats[i, 0] = d.params.repetition_penalty if recent else 1.0
            floats[i, 1] = d.params.resolved_temperature
        dev = torch.from_numpy(host).to(self.device)
        recent = dev[:, :RECENT_TOKENS].contiguous()
        scalars = dev[:, RECENT_TOKENS:].t().contiguous().view(torch.float32)
        return ops.repetition_penalty(logits.clone(), recent, scalars[0], scalars[1])
