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
from typing import Any, Mapping, Optional, Sequence, Tuple, Union


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


PartSpec = Union[NormSpec, MixerSpec, FeedForwardSpec]


class LayerSpec:
    """One block: its parts by role, in the order the arrangement names them, and how they are arranged.
    `"pre_norm"` (x += mixer(mixer_norm(x)); x += ffn(ffn_norm(x))) takes the four roles `mixer_norm`,
    `mixer`, `ffn_norm`, `ffn`, which may be given in that order as positional arguments; another
    arrangement names whatever roles it wants through `parts` (one norm and two bodies, a block
    without a feed-forward, two mixers, norms after the bodies), and any number of them may be
    mixers with caches or state of their own."""
    PRE_NORM_ROLES = ("mixer_norm", "mixer", "ffn_norm", "ffn")

    def __init__(self, name: str, arrangement: str, mixer_norm: Optional[NormSpec] = None, mixer: Optional[MixerSpec] = None,
                 ffn_norm: Optional[NormSpec] = None, ffn: Optional[FeedForwardSpec] = None,
                 parts: Optional[Sequence[Tuple[str, PartSpec]]] = None):
        self.name = name                    # checkpoint prefix, e.g. "model.layers.3"
        self.arrangement = arrangement
        if parts is None:
            parts = [(r, p) for r, p in zip(self.PRE_NORM_ROLES, (mixer_norm, mixer, ffn_norm, ffn)) if p is not None]
        elif any(p is not None for p in (mixer_norm, mixer, ffn_norm, ffn)):
            raise ValueError("a layer's parts are given either by role (`parts`) or as the four of a pre-norm block")
        self.parts: Tuple[Tuple[str, PartSpec], ...] = tuple((str(r), p) for r, p in parts)
        roles = [r for r, _ in self.parts]
        if len(set(roles)) != len(roles):
            raise ValueError(f"layer {name!r} names a role twice: {roles}")

    def part(self, role: str) -> PartSpec:
        for r, p in self.parts:
            if r == role:
                return p
        raise KeyError(f"layer {self.name!r} has no part {role!r}; it has {[r for r, _ in self.parts]}")

    # the four roles of a pre-norm block, by name
    mixer_norm = property(lambda self: self.part("mixer_norm"))
    mixer = property(lambda self: self.part("mixer"))
    ffn_norm = property(lambda self: self.part("ffn_norm"))
    ffn = property(lambda self: self.part("ffn"))

    def __eq__(self, other) -> bool:
        return isinstance(other, LayerSpec) and (self.name, self.arrangement, self.parts) == (other.name, other.arrangement, other.parts)

    def __repr__(self) -> str:
        return f"LayerSpec({self.name!r}, {self.arrangement!r}, parts={self.parts!r})"


@dataclass(frozen=True)
class ModelSpec:
    """A whole decoder.  `layers` are the distinct layers (each owns weights and, if its
    mixers need them, caches); `order` is the list of layer indices in the order they run:
    it may name a layer twice.  A mixer whose params carry `kv_source` reads the cache of
    that layer (of its first mixer that owns one) instead of owning one."""
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
