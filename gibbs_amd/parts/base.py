"""Interfaces of the parts a layer is put together from, and the registries that map a
spec's `kind` to the class that implements it.

A part is built from its spec alone (sizes and constants are the spec's parameters), declares
the checkpoint tensors it reads, is bound to loaded weights, and lays itself down in the native
plan of the model's step (`emit`, parts/native.py).  No part knows which model it is in.  To add
a part: subclass the interface, decorate the class with the matching `register_*`, and name its
kind in a spec; nothing else in the framework changes.

  Norm            forward(x, delta, rows) -> normed rows in the activation dtype (adds delta first)
  PositionEncoding  tables and parameters that a mixer hands to its kernels
  Mixer           forward(h, batch, cache) -> delta [N, hidden] (or float32 parts [S, N, hidden]
                  that are added in order); may ask for cache pages (`cache_need`) and
                  per-request state of fixed size (`state_needs`)
  FeedForward     forward(h, batch) -> delta [N, hidden]
  Block           emit(plan, caches): the arrangement of a layer's parts, as operations of the plan

A part written with tensor operations implements `forward` and nothing else: the base class's
`emit` lays it down as a callback of the native step.  A part with kernels of its own in the
library overrides `emit` (the built-in ones do); its `forward` then runs the part alone through a
small plan of its own, the same native code that a whole step takes.

Optional fast-path hooks: a norm may offer `fold_gain()` (hand its gain over to be multiplied into
the following matrices), a mixer or feed-forward `fold_input_gain(gain)` and `pack_matrices()`.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, Dict, List, Mapping, Optional, Sequence, Type

import torch

from ..cache.needs import CacheNeed, StateNeed
from ..config.spec import FeedForwardSpec, LayerSpec, MixerSpec, NormSpec, PositionSpec
from ..weights.loader import TensorDecl, WeightStore


@dataclass
class Runtime:
    """What a part needs to know about the run it is bound into."""
    device: torch.device
    act_dtype: torch.dtype          # activations and cache pages: bfloat16, or float32 for the 32-bit path
    max_positions: int = 0          # positions a request can reach (tables over positions are sized by it); 0: unknown
    shared: Dict = field(default_factory=dict)   # what parts of one model derive once and share (tables)
    # bfloat16 only: norm gains are multiplied into the matrices that read the normed rows, and steps of
    # up to `fused_decode_rows` single decoded tokens take the parts' fused decode kernels (0: never)
    fold_gains: bool = True
    fused_decode_rows: int = 64


class Part:
    def tensor_decls(self) -> List[TensorDecl]:
        return []

    def bind(self, weights: WeightStore, rt: Runtime) -> None:
        """Takes its tensors from the store and prepares the layouts its kernels want."""
        self.rt = rt

    def matrices(self) -> List[torch.Tensor]:
        """The matrices [out, in] that every row of a step is multiplied with (what a decode step
        has to stream, and 2 * numel flops per row)."""
        return []

    def product_shapes(self) -> List[tuple]:
        """(out, in) of the matrix products that every row of a step goes through, known from the
        sizes alone (before any weights are bound)."""
        return []

    def small_tensors(self) -> List[torch.Tensor]:
        """Gains, biases, taps and tables that a step also reads."""
        return []

    def pack_matrices(self) -> None:
        """Called once the matrices have their final values (gains folded in): a part may keep
        copies in the order its few-row kernels read fastest (`ops.PackedWeight`)."""


def _solo_plan(rt: Runtime, hidden: int):
    """A plan of one part's own, for running it alone."""
    from .native import NativePlan
    return NativePlan(rt, hidden)


class Norm(Part):
    def __init__(self, spec: NormSpec, width: int):
        self.spec, self.width = spec, width

    def emit(self, plan) -> int:
        """Lays the norm down in `plan`; returns its number there.  Default: a callback to `forward`."""
        if type(self).forward is Norm.forward:
            raise NotImplementedError(f"{type(self).__name__} has neither `forward` nor `emit`")
        return plan.host_norm(self.forward)

    def forward(self, x: torch.Tensor, delta: Optional[torch.Tensor], rows: Optional[torch.Tensor] = None,
                n_rows: Optional[int] = None) -> torch.Tensor:
        """x (float32 residual stream) += delta (if given and all rows are normed); returns norm(x)
        in the activation dtype.  With `rows` only those rows (of x + delta) are normed.  `delta` is
        [N, width] in the activation dtype, or float32 [S, N, width]: parts that are added in
        ascending s (a product that was split over its inner dimension).  (A norm with `emit` of its
        own runs alone through a plan of one part.)"""
        if type(self).emit is Norm.emit:
            raise NotImplementedError(f"{type(self).__name__} has neither `forward` nor `emit`")
        solo = getattr(self, "_solo", None)
        if solo is None:
            plan = _solo_plan(self.rt, self.width)
            solo = self._solo = (plan, self.emit(plan))
        return solo[0].norm_forward(solo[1], x, delta, rows, n_rows)


@dataclass
class Rotation:
    """A rotation of q and k by position that the attention kernels apply themselves."""
    inv_freq: torch.Tensor                 # float32 [rotary_dim / 2]
    rotary_dim: int
    variant: str                           # "half_split": pairs (j, j + rotary_dim/2); "interleaved": pairs (2j, 2j+1)
    cos_sin: Optional[torch.Tensor] = None  # [positions, rotary_dim / 2, 2] of the first positions, or None


class PositionEncoding(Part):
    """How positions enter an attention mixer.  An encoding answers in one (or more) of three ways,
    and the mixer asks in this order:

      rotation()        a `Rotation`: the kernels rotate q and k themselves (all fast paths stay open);
      apply(q, k, batch)  anything else done to q and k in place before k is cached (the mixer then
                        takes its general path: norm, this hook, cache write, attention);
      score_slopes(heads)  float32 [heads]: slope[h] * (key position - query position) is added to the
                        scores (a linear bias over the distance; the plain attention kernel takes it).

    An encoding that answers none of them leaves q, k and the scores alone."""

    def __init__(self, spec: PositionSpec, head_dim: int):
        self.spec, self.head_dim = spec, head_dim

    def rotation(self) -> Optional[Rotation]:
        return None

    def apply(self, q: torch.Tensor, k: Optional[torch.Tensor], batch) -> None:
        """q: [N, heads, head_dim], k: [N, kv_heads, head_dim] (None for a mixer that reads another
        layer's cache): views of the step's rows, after the q/k norm, changed in place.  `batch.pos`
        holds every row's position."""

    def score_slopes(self, heads: int) -> Optional[torch.Tensor]:
        return None

    def transforms_rows(self) -> bool:
        """Whether `apply` does anything (the mixer skips the hook's extra passes otherwise)."""
        return type(self).apply is not PositionEncoding.apply


class Mixer(Part):
    def __init__(self, spec: MixerSpec, hidden: int, layer_index: int):
        self.spec, self.hidden, self.layer_index = spec, hidden, layer_index

    def cache_need(self) -> Optional[CacheNeed]:
        """Paged keys/values this mixer owns (None: none)."""
        return None

    def kv_source(self) -> Optional[int]:
        """Index of the layer whose pages this mixer reads instead of owning pages."""
        return None

    def state_needs(self) -> Sequence[StateNeed]:
        return ()

    def attention_flops(self, keys: float) -> float:
        """Flops that grow with the keys the step's rows see (`keys`: their sum over the rows), beside
        the matrix products: scores and weighted values of an attention; 0 for a mixer without."""
        return 0.0

    def emit(self, plan, cache) -> int:
        """Lays the mixer down in `plan` over the cache view `cache`; returns its number there.
        Default: a callback to `forward`."""
        if type(self).forward is Mixer.forward:
            raise NotImplementedError(f"{type(self).__name__} has neither `forward` nor `emit`")
        return plan.host_body(lambda h, batch: self.forward(h, batch, cache), None if cache.kpages is None else cache.group)

    def forward(self, h: torch.Tensor, batch, cache) -> torch.Tensor:
        """The delta of the normed rows h [N, hidden] (a mixer with `emit` of its own runs alone
        through a plan of one part, kept per cache view)."""
        if type(self).emit is Mixer.emit:
            raise NotImplementedError(f"{type(self).__name__} has neither `forward` nor `emit`")
        solos = self.__dict__.setdefault("_solos", {})
        solo = solos.get(id(cache))
        if solo is None:
            plan = _solo_plan(self.rt, self.hidden)
            solo = solos[id(cache)] = (plan, self.emit(plan, cache), cache)
        return solo[0].body_forward(solo[1], h.contiguous(), batch)


class FeedForward(Part):
    def __init__(self, spec: FeedForwardSpec, hidden: int):
        self.spec, self.hidden = spec, hidden

    def emit(self, plan) -> int:
        """Lays the feed-forward down in `plan`; returns its number there.  Default: a callback to `forward`."""
        if type(self).forward is FeedForward.forward:
            raise NotImplementedError(f"{type(self).__name__} has neither `forward` nor `emit`")
        return plan.host_body(lambda h, batch: self.forward(h, batch))

    def forward(self, h: torch.Tensor, batch) -> torch.Tensor:
        if type(self).emit is FeedForward.emit:
            raise NotImplementedError(f"{type(self).__name__} has neither `forward` nor `emit`")
        solo = getattr(self, "_solo", None)
        if solo is None:
            plan = _solo_plan(self.rt, self.hidden)
            solo = self._solo = (plan, self.emit(plan))
        return solo[0].body_forward(solo[1], h.contiguous(), batch)


def build_part(spec, hidden: int, layer_index: int) -> Part:
    """The part that a spec of any of the layer's kinds describes."""
    if isinstance(spec, NormSpec):
        return build_norm(spec, hidden)
    if isinstance(spec, MixerSpec):
        return build_mixer(spec, hidden, layer_index)
    if isinstance(spec, FeedForwardSpec):
        return build_feed_forward(spec, hidden)
    raise TypeError(f"a layer's parts are norms, mixers and feed-forwards, not {type(spec).__name__}")


class Block(Part):
    """One layer: its parts by role, as the layer's spec names them (any number of norms, mixers and
    feed-forwards), and their arrangement, which a subclass lays down in `emit`."""

    def __init__(self, spec: LayerSpec, hidden: int, layer_index: int):
        self.spec, self.hidden = spec, hidden
        self.named: Dict[str, Part] = {role: build_part(ps, hidden, layer_index) for role, ps in spec.parts}

    def __getattr__(self, role: str) -> Part:
        """`block.mixer`, `block.ffn_norm`, ...: the part of that role."""
        named = self.__dict__.get("named", {})
        if role in named:
            return named[role]
        raise AttributeError(f"{type(self).__name__} has no attribute or part {role!r}")

    def parts(self) -> List[Part]:
        return list(self.named.values())

    def mixers(self) -> Dict[str, Mixer]:
        """The parts that may own a cache or state, by role, in the spec's order."""
        return {role: p for role, p in self.named.items() if isinstance(p, Mixer)}

    def tensor_decls(self) -> List[TensorDecl]:
        return [d for p in self.parts() for d in p.tensor_decls()]

    def bind(self, weights: WeightStore, rt: Runtime) -> None:
        self.rt = rt
        for p in self.parts():
            p.bind(weights, rt)

    def matrices(self) -> List[torch.Tensor]:
        return [m for p in self.parts() for m in p.matrices()]

    def product_shapes(self) -> List[tuple]:
        return [m for p in self.parts() for m in p.product_shapes()]

    def small_tensors(self) -> List[torch.Tensor]:
        return [m for p in self.parts() for m in p.small_tensors()]

    def attention_flops(self, keys: float) -> float:
        return sum(m.attention_flops(keys) for m in self.mixers().values())

    def emit(self, plan, caches: Mapping[str, object]) -> None:
        """Lays the block down in `plan`: its parts (`part.emit`) and the operations that arrange them
        (`plan.half`, or `plan.normed` / `plan.apply` / `plan.add` / `plan.drop` in any order).
        `caches[role]`: the cache view of the mixer of that role."""
        raise NotImplementedError

    def forward(self, x: torch.Tensor, batch, caches: Mapping[str, object]) -> torch.Tensor:
        """The block alone on the residual rows x [N, hidden] (float32, changed in place): through a plan
        that holds this block only (kept per set of cache views).  Returns x."""
        solos = self.__dict__.setdefault("_solos", {})
        key = tuple(id(c) for c in caches.values())
        solo = solos.get(key)
        if solo is None:
            from .native import NativePlan
            plan = NativePlan(self.rt, self.hidden)
            self.emit(plan, caches)
            solo = solos[key] = (plan, dict(caches))
        solo[0].step(batch, x_in=x, first_op=0, n_ops=solo[0].op_count(), settle=True)
        return x


# --------------------------------------------------------------------------- registries
NORMS: Dict[str, Type[Norm]] = {}
POSITIONS: Dict[str, Type[PositionEncoding]] = {}
MIXERS: Dict[str, Type[Mixer]] = {}
FEED_FORWARDS: Dict[str, Type[FeedForward]] = {}
ARRANGEMENTS: Dict[str, Type[Block]] = {}


def _register(table: Dict[str, type], kind: str) -> Callable[[type], type]:
    def deco(cls: type) -> type:
        table[kind] = cls
        return cls
    return deco


def register_norm(kind: str): return _register(NORMS, kind)
def register_position(kind: str): return _register(POSITIONS, kind)
def register_mixer(kind: str): return _register(MIXERS, kind)
def register_feed_forward(kind: str): return _register(FEED_FORWARDS, kind)
def register_arrangement(kind: str): return _register(ARRANGEMENTS, kind)


def _lookup(table: Dict[str, type], kind: str, what: str) -> type:
    if kind not in table:
        raise KeyError(f"no {what} of kind {kind!r} is registered; known: {sorted(table)}")
    return table[kind]


def build_norm(spec: NormSpec, width: int) -> Norm:
    return _lookup(NORMS, spec.kind, "norm")(spec, width)


def build_position(spec: Optional[PositionSpec], head_dim: int) -> Optional[PositionEncoding]:
    if spec is None or spec.kind == "none":
        return None
    return _lookup(POSITIONS, spec.kind, "position encoding")(spec, head_dim)


def build_mixer(spec: MixerSpec, hidden: int, layer_index: int) -> Mixer:
    return _lookup(MIXERS, spec.kind, "mixer")(spec, hidden, layer_index)


def build_feed_forward(spec: FeedForwardSpec, hidden: int) -> FeedForward:
    return _lookup(FEED_FORWARDS, spec.kind, "feed-forward")(spec, hidden)


def build_block(spec: LayerSpec, hidden: int, layer_index: int) -> Block:
    return _lookup(ARRANGEMENTS, spec.arrangement, "block arrangement")(spec, hidden, layer_index)
