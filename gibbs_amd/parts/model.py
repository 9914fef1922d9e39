"""A decoder put together from a `ModelSpec`: token table, blocks in the spec's run order, final
norm and head (arch/families/lfm2.json5:66-95,
arch/lib/transformer.json5:170-198).

The model owns structure and weights; its step is the native plan that its blocks lay down
(parts/native.py).  Only the rows whose logits are wanted go through the final norm and the head:
the gather comes before the norm, as in the reference's `last_row` (transformer.json5:177-192).
"""
from __future__ import annotations

from typing import List, Optional, Sequence, Tuple

import torch

from .. import ops
from ..cache.needs import CacheNeed, StateNeed
from ..config.spec import ModelSpec
from ..weights.loader import TensorDecl, WeightStore
from .base import Block, Part, Runtime, build_block, build_norm


class DecoderModel(Part):
    def __init__(self, spec: ModelSpec):
        self.spec = spec
        self.blocks: List[Block] = [build_block(ls, spec.hidden, i) for i, ls in enumerate(spec.layers)]
        self.final_norm = build_norm(spec.final_norm, spec.hidden)
        for i in spec.order:
            if not 0 <= i < len(self.blocks):
                raise ValueError(f"layer order names layer {i}; the model has {len(self.blocks)}")
        for i, b in enumerate(self.blocks):
            for mixer in b.mixers().values():
                src = mixer.kv_source()
                if src is None:
                    continue
                if not 0 <= src < len(self.blocks) or self._cache_owner_role(src) is None:
                    raise ValueError(f"layer {i} reads the cache of layer {src}, which owns none")
                first_use = spec.order.index(i) if i in spec.order else -1
                if first_use >= 0 and src not in spec.order[:first_use]:
                    raise ValueError(f"layer {i} runs before layer {src}, whose cache it reads")

    def _cache_owner_role(self, layer: int) -> Optional[str]:
        """The role of the first mixer of `layer` that owns cache pages."""
        return next((role for role, m in self.blocks[layer].mixers().items() if m.cache_need() is not None), None)

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

    # Caches belong to the mixers of runs (entries of the run order), not to layers: a layer that the
    # order names twice shares its weights between both runs, but each run caches its own keys,
    # values and state.  `cache_owners` lists them, (run, role) in the order they run; what the cache
    # manager calls a layer is an entry of this list.
    def cache_owners(self) -> List[Tuple[int, str]]:
        return [(run, role) for run, i in enumerate(self.spec.order) for role in self.blocks[i].mixers()]

    def _mixer(self, owner: Tuple[int, str]):
        return self.blocks[self.spec.order[owner[0]]].mixers()[owner[1]]

    def cache_needs(self) -> List[Optional[CacheNeed]]:
        return [self._mixer(o).cache_need() for o in self.cache_owners()]

    def state_needs(self) -> List[Sequence[StateNeed]]:
        return [tuple(self._mixer(o).state_needs()) for o in self.cache_owners()]

    def kv_sources(self) -> List[Optional[int]]:
        """For each cache owner, the earlier owner whose pages it reads (the page-owning mixer of the
        latest run of the layer that its mixer names as `kv_source`), or None."""
        owners = self.cache_owners()
        out: List[Optional[int]] = []
        for run, role in owners:
            src = self._mixer((run, role)).kv_source()
            if src is None:
                out.append(None)
                continue
            src_run = max(j for j in range(run) if self.spec.order[j] == src)
            out.append(owners.index((src_run, self._cache_owner_role(src))))
        return out

    def bind(self, weights: WeightStore, rt: Runtime) -> None:
        self.rt = rt
        self.table = weights[self.spec.embedding]
        self.head = weights[self.spec.head] if self.spec.head is not None else self.table
        self.head_packed = ops.PackedWeight(self.head) if rt.act_dtype == torch.bfloat16 else None
        self.final_norm.bind(weights, rt)
        for b in self.blocks:
            b.bind(weights, rt)
