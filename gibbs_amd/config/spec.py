"""Architecture-neutral description of a decoder: what each layer is made of.

An architecture's typed configuration (for instance `Lfm2Config`) turns its own
config.json keys into a `ModelSpec`.  Everything below the configuration (parts,
cache manager, step function) reads only these specs, so a part never knows which
model it sits in, and one model may use different mixers and feed-forwards in
different layers.  Every size and constant that config.json gives travels here as
a field; none is written into the code of a part.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Mapping, Optional, Tuple


@dataclass(frozen=True)
class NormSpec:
    """A normalisation over the last axis. `kind` selects the part (`"rms"`)."""
    kind: str
    eps: float
    weight: str                     # tensor name of the gain


@dataclass(frozen=True)
class PositionSpec:
    """A position encoding applied inside a mixer (`"rope"`, `"none"`, or one that a
    test or another architecture registers).  `tensors` names the checkpoint tensors of an
    encoding that has any (a learned table)."""
    kind: str
    params: Mapping[str, Any] = field(default_factory=dict)
    tensors: Mapping[str, str] = field(default_factory=dict)


@dataclass(frozen=True)
class MixerSpec:
    """The token mixer of a layer (`"attention"`, `"short_conv"`, ...).  `params` holds
    the sizes and constants of that kind; `tensors` maps the part's own tensor roles
    (for instance `"q_proj"`) to checkpoint names."""
    kind: str
    params: Mapping[str, Any]
    tensors: Mapping[str, str]
    position: Optional[PositionSpec] = None


@dataclass(frozen=True)
class FeedForwardSpec:
    """The feed-forward of a layer (`"glu"` dense here; an expert feed-forward would be
    another kind with its router and expert tensors)."""
    kind: str
    params: Mapping[str, Any]
    tensors: Mapping[str, str]


@dataclass(frozen=True)
class LayerSpec:
    """One block: how norm, mixer and feed-forward are arranged (`"pre_norm"`:
    x += mixer(norm(x)); x += ffn(norm(x)))."""
    name: str                       # checkpoint prefix, e.g. "model.layers.3"
    arrangement: str
    mixer_norm: NormSpec
    mixer: MixerSpec
    ffn_norm: NormSpec
    ffn: FeedForwardSpec


@dataclass(frozen=True)
class ModelSpec:
    """A whole decoder.  `layers` are the distinct layers (each owns weights and, if its
    mixer needs one, a cache); `order` is the list of layer indices in the order they run:
    it may name a layer twice.  A mixer whose params carry `kv_source` reads the cache of
    that layer instead of owning one."""
    architecture: str
    hidden: int
    vocab: int
    layers: Tuple[LayerSpec, ...]
    order: Tuple[int, ...]
    embedding: str                  # tensor name of the token table
    final_norm: NormSpec
    head: Optional[str]             # tensor name of an untied head; None = tied to the table
    max_position: int
    eos_token_ids: Tuple[int, ...] = ()
    bos_token_id: Optional[int] = None
