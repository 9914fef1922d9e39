"""Interfaces of the parts a layer is put together from, and the registries that map a
spec's `kind` to the class that implements it.

A part is built from its spec alone (sizes and constants are the spec's parameters), declares
the checkpoint tensors it reads, and is later bound to loaded weights.  No part knows which
model it is in.  To add a part: subclass the interface, decorate the class with the matching
`register_*`, and name its kind in a spec; nothing else in the framework changes.

  Norm            forward(x, delta, rows) -> normed rows in the activation dtype (adds delta first)
  PositionEncoding  tables and parameters that a mixer hands to its kernels
  Mixer           forward(h, batch, cache) -> delta [N, hidden] (or float32 parts [S, N, hidden]
                  that the next norm adds in order); may ask for cache pages
                  (`cache_need`) and per-request state of fixed size (`state_needs`)
  FeedForward     forward(h, batch) -> delta [N, hidden]
  Block           forward(stream, batch, cache) -> stream (arrangement of the above)

Optional fast-path hooks (a part without them simply takes the general path): a norm may offer
`fold_gain()` (hand its gain over to be multiplied into the following matrices), a mixer or
feed-forward `fold_input_gain(gain)` and `decode_fused(stream, norm_eps, batch[, cache])`, which
runs norm + part + residual add for a step of single decoded tokens in a few fused kernels.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional, Sequence, Type

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


@dataclass
class Stream:
    """The residual stream between blocks.  `x` is float32 [N, hidden].  `pending` is a delta that
    has not been added yet (the next norm adds it as it reads x).  `mirror`, when kept, is
    bfloat16(x) with nothing pending: what the fused decode products read as their input."""
    x: torch.Tensor
    pending: Optional[torch.Tensor] = None
    mirror: Optional[torch.Tensor] = None

    # What every arrangement does with the stream, so that none has to know how deltas travel:
    def normed(self, norm: "Norm", rows: Optional[torch.Tensor] = None, n_rows: Optional[int] = None) -> torch.Tensor:
        """norm(x + what is pending) in the activation type.  All rows: the pending delta is added
        into x on the way (one kernel).  With `rows`, only those rows are normed and x stays as it is."""
        h = norm.forward(self.x, self.pending, rows, n_rows)
        if rows is None and self.pending is not None:
            self.pending, self.mirror = None, None
        return h

    def add(self, delta: torch.Tensor) -> None:
        """x += delta, lazily: the delta stays pending until the next `normed` or `add` (a delta is
        [N, hidden] in the activation type, or float32 partial sums [S, N, hidden])."""
        self.settle()
        self.pending, self.mirror = delta, None

    def settle(self) -> None:
        """Adds what is pending into x now."""
        if self.pending is not None:
            from .. import ops
            ops.residual_add(self.x, self.pending)
            self.pending, self.mirror = None, None

    def with_mirror(self) -> "Stream":
        """Settles the stream and makes sure that `mirror` = bfloat16(x) exists (one kernel for both)."""
        if self.pending is not None or self.mirror is None:
            from .. import ops
            mirror = torch.empty(self.x.shape, dtype=torch.bfloat16, device=self.x.device)
            ops.residual_add(self.x, self.pending, mirror)
            self.pending, self.mirror = None, mirror
        return self


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


class Norm(Part):
    def __init__(self, spec: NormSpec, width: int):
        self.spec, self.width = spec, width

    def forward(self, x: torch.Tensor, delta: Optional[torch.Tensor], rows: Optional[torch.Tensor] = None,
                n_rows: Optional[int] = None) -> torch.Tensor:
        """x (float32 residual stream) += delta (if given and all rows are normed); returns norm(x)
        in the activation dtype.  With `rows` only those rows (of x + delta) are normed.  `delta` is
        [N, width] in the activation dtype, or float32 [S, N, width]: parts that are added in
        ascending s (a product that was split over its inner dimension)."""
        raise NotImplementedError


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

    def forward(self, h: torch.Tensor, batch, cache) -> torch.Tensor:
        raise NotImplementedError


class FeedForward(Part):
    def __init__(self, spec: FeedForwardSpec, hidden: int):
        self.spec, self.hidden = spec, hidden

    def forward(self, h: torch.Tensor, batch) -> torch.Tensor:
        raise NotImplementedError


class Block(Part):
    """One layer: an arrangement of two norms, a mixer and a feed-forward."""

    def __init__(self, spec: LayerSpec, hidden: int, layer_index: int):
        self.spec = spec
        self.mixer_norm = build_norm(spec.mixer_norm, hidden)
        self.mixer = build_mixer(spec.mixer, hidden, layer_index)
        self.ffn_norm = build_norm(spec.ffn_norm, hidden)
        self.ffn = build_feed_forward(spec.ffn, hidden)

    def parts(self) -> List[Part]:
        return [self.mixer_norm, self.mixer, self.ffn_norm, self.ffn]

    def tensor_decls(self) -> List[TensorDecl]:
        return [d for p in self.parts() for d in p.tensor_decls()]

    def bind(self, weights: WeightStore, rt: Runtime) -> None:
        self.rt = rt
        for p in self.parts():
            p.bind(weights, rt)

    def matrices(self) -> List[torch.Tensor]:
        return [m for p in self.parts() for m in p.matrices()]

    def small_tensors(self) -> List[torch.Tensor]:
        return [m for p in self.parts() for m in p.small_tensors()]

    def forward(self, stream: Stream, batch, cache) -> Stream:
        """Runs the block on the residual stream (updated in place) and returns it, with the
        block's last delta either added or left pending for the next norm."""
        raise NotImplementedError


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
