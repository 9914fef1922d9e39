"""A decoder put together from a `ModelSpec`: token table, blocks in the spec's run order, final
norm and head (arch/families/lfm2.json5:66-95,
arch/lib/transformer.json5:170-198).

Only the rows whose logits are wanted go through the final norm and the head: the gather comes
before the norm, as in the reference's `last_row` (transformer.json5:177-192).
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import torch

from .. import ops
from ..cache.needs import CacheNeed, StateNeed
from ..config.spec import ModelSpec
from ..ops.linear import linear
from ..weights.loader import TensorDecl, WeightStore
from .base import Block, Part, Runtime, Stream, build_block, build_norm
from .block import fused_decode_step


class DecoderModel(Part):
    def __init__(self, spec: ModelSpec):
        self.spec = spec
        self.blocks: List[Block] = [build_block(ls, spec.hidden, i) for i, ls in enumerate(spec.layers)]
        self.final_norm = build_norm(spec.final_norm, spec.hidden)
        for i in spec.order:
            if not 0 <= i < len(self.blocks):
                raise ValueError(f"layer order names layer {i}; the model has {len(self.blocks)}")
        for i, b in enumerate(self.blocks):
            src = b.mixer.kv_source()
            if src is not None:
                if not 0 <= src < len(self.blocks) or self.blocks[src].mixer.cache_need() is None:
                    raise ValueError(f"layer {i} reads the cache of layer {src}, which owns none")
                first_use = spec.order.index(i) if i in spec.order else -1
                if first_use >= 0 and src not in spec.order[:first_use]:
                    raise ValueError(f"layer {i} runs before layer {src}, whose cache it reads")

    # ------------------------------------------------------------------ what the model asks for
    def tensor_decls(self) -> List[TensorDecl]:
        s = self.spec
        decls = [TensorDecl(s.embedding, (s.vocab, s.hidden))]
        decls += self.final_norm.tensor_decls()
        for b in self.blocks:
            decls += b.tensor_decls()
        if s.head is not None:
            decls.append(TensorDecl(s.head, (s.vocab, s.hidden)))
        return decls

    # Caches belong to runs (entries of the run order), not to layers: a layer that the order
    # names twice shares its weights between both runs, but each run caches its own keys,
    # values and state.
    def cache_needs(self) -> List[Optional[CacheNeed]]:
        return [self.blocks[i].mixer.cache_need() for i in self.spec.order]

    def state_needs(self) -> List[Sequence[StateNeed]]:
        return [tuple(self.blocks[i].mixer.state_needs()) for i in self.spec.order]

    def kv_source_runs(self) -> List[Optional[int]]:
        """For each run, the earlier run whose pages it reads (the latest run of the layer that
        its mixer names as `kv_source`), or None."""
        out: List[Optional[int]] = []
        for run, i in enumerate(self.spec.order):
            src = self.blocks[i].mixer.kv_source()
            out.append(None if src is None else max(j for j in range(run) if self.spec.order[j] == src))
        return out

    def bind(self, weights: WeightStore, rt: Runtime) -> None:
        self.rt = rt
        self.table = weights[self.spec.embedding]
        self.head = weights[self.spec.head] if self.spec.head is not None else self.table
        self.head_packed = ops.PackedWeight(self.head) if rt.act_dtype == torch.bfloat16 else None
        self.final_norm.bind(weights, rt)
        for b in self.blocks:
            b.bind(weights, rt)

    # ------------------------------------------------------------------ one step
    def forward(self, batch, caches) -> Optional[torch.Tensor]:
        """Runs the batch's rows through every layer from the cache (`caches[run]` is the view of
        run number `run` of the layer order); returns float32 logits [len(logit_rows), vocab]
        (None if no logits are wanted)."""
        mirror = None
        if fused_decode_step(self.rt, batch):
            # a step of decoded tokens: the fused kernels read the stream's bfloat16 mirror
            mirror = torch.empty((batch.n_rows, self.spec.hidden), dtype=torch.bfloat16, device=self.rt.device)
        stream = Stream(ops.embed(self.table, batch.ids, batch.n_rows, mirror=mirror), None, mirror)
        for run, i in enumerate(self.spec.order):
            stream = self.blocks[i].forward(stream, batch, caches[run])
        if batch.n_logits == 0:
            return None
        h = stream.normed(self.final_norm, batch.logit_rows, batch.n_logits)
        return linear(h, self.head, out_dtype=torch.float32, packed=self.head_packed)
