"""The engine: a model bound to its weights and cache, and the one step function.

`step(entries)` runs exactly the tokens it is given, as one batch, from the cache that earlier
steps left, and returns the logits at the wanted places.  The reference's counterpart is
`NativeLm::forward(tokens, start_pos, state)` for one sequence
(/root/reference/src/model/native.rs:78-83, /root/reference/src/runtime/lm.rs:513-583); here a
step takes any mix of prompt portions and decoded tokens of several requests.  Its guards are
the reference's (lm.rs:528-544): no empty token list, no position beyond the context limit.
"""
from __future__ import annotations

import os
from typing import Dict, Hashable, List, Optional, Sequence

import numpy as np
import torch

from ..cache import CacheManager, DeviceCache
from ..config import config_from_dict, read_config_json
from ..config.base import ArchConfig
from ..ops.lib import KernelError, library
from ..parts import DecoderModel, Runtime
from ..weights import WeightStore, load_weights, table_of
from .batch import BatchStager, Entry, StepBatch

DEFAULT_PAGE_SIZE = 16      # tokens per cache page, the reference's block size (/root/reference/src/kv/mod.rs:6)
DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32}


class OutOfPages(RuntimeError):
    """The step needs more cache pages (or a slot) than are free; nothing was changed."""


class StepError(ValueError):
    """The step's entries cannot be run (empty tokens, bad ids, context limit, unknown request)."""


class Engine:
    def __init__(self, model_dir: Optional[str] = None, *, dtype: str = "bfloat16", max_tokens: int = 8192,
                 max_requests: int = 8, page_size: int = DEFAULT_PAGE_SIZE, device: str = "cuda:0", arch: Optional[str] = None,
                 ctx: Optional[int] = None, config: Optional[ArchConfig] = None,
                 weights: Optional[WeightStore] = None):
        """`model_dir`: a folder with config.json and model.safetensors (the model class is chosen
        by config.json).  `max_tokens`: tokens the cache pool holds (each request's count rounded
        up to whole pages).  `ctx`: context limit, default config.json's max_position_embeddings.
        `config` + `weights` may stand in for a folder (weights already on the device)."""
        if not torch.cuda.is_available():
            raise KernelError("no GPU: this engine has no CPU path")
        if dtype not in DTYPES:
            raise ValueError(f"dtype {dtype!r} is not one of {sorted(DTYPES)}")
        library()                                   # fail now, loudly, if the kernels are missing
        self.device = torch.device(device)
        torch.cuda.set_device(self.device)
        self.dtype = DTYPES[dtype]
        if config is None:
            cfg = read_config_json(model_dir)
            config = config_from_dict(cfg, tensors=table_of(model_dir), arch=arch)
        self.config = config
        self.spec = config.model_spec()
        self.model = DecoderModel(self.spec)
        if weights is None:
            weights = load_weights(model_dir, self.model.tensor_decls(), self.dtype, self.device)
        self.page_size = page_size
        self.ctx_limit = int(ctx) if ctx else self.spec.max_position
        num_pages = max(1, -(-max_tokens // page_size))
        self.rt = Runtime(self.device, self.dtype, max_positions=min(self.ctx_limit, num_pages * page_size))
        self.model.bind(weights, self.rt)
        self.weight_bytes = weights.nbytes()
        del weights

        self.cache = CacheManager(self.model.cache_needs(), self.model.state_needs(), page_size, num_pages,
                                  max_requests)
        self.device_cache = DeviceCache(self.cache, self.dtype, self.device)
        self._views = [self.device_cache.layer_view(run, src)
                       for run, src in enumerate(self.model.kv_source_runs())]
        self._stager = BatchStager(self.device)

    # ------------------------------------------------------------------ requests
    def admit(self, rid: Hashable) -> bool:
        return self.cache.admit(rid)

    def release(self, rid: Hashable) -> None:
        """A request ended: its pages and slot are given back."""
        self.cache.release(rid)

    def cached_tokens(self, rid: Hashable) -> int:
        return self.cache.tokens(rid)

    # ------------------------------------------------------------------ the step function
    def prepare(self, entries: Sequence[Entry]) -> StepBatch:
        """Checks the entries, takes slots and pages for them and stages the batch's metadata."""
        if not entries:
            raise StepError("a step needs at least one entry")
        seen = set()
        vocab = self.spec.vocab
        token_arrays = []
        for e in entries:
            if e.rid in seen:
                raise StepError(f"request {e.rid!r} appears twice in one step")
            seen.add(e.rid)
            if len(e.tokens) == 0:
                raise StepError(f"request {e.rid!r}: no tokens")
            toks = np.asarray(e.tokens, dtype=np.int64)
            token_arrays.append(toks)
            if toks.min() < 0 or toks.max() >= vocab:
                bad = int(toks[(toks < 0) | (toks >= vocab)][0])
                raise StepError(f"request {e.rid!r}: token id {bad} outside the vocabulary (0..{vocab - 1})")
            if any(not 0 <= w < len(e.tokens) for w in e.want):
                raise StepError(f"request {e.rid!r}: wanted place outside its {len(e.tokens)} tokens")
            before = self.cache.tokens(e.rid) if e.rid in self.cache else 0
            if before + len(e.tokens) > self.ctx_limit:
                raise StepError(f"request {e.rid!r}: {before + len(e.tokens)} tokens exceed the context limit {self.ctx_limit}")
        # slots and pages: all or nothing for the whole step
        admitted, reserved = [], []
        try:
            for e in entries:
                if e.rid not in self.cache:
                    if not self.cache.admit(e.rid):
                        raise OutOfPages(f"no free slot for request {e.rid!r} ({self.cache.max_requests} live)")
                    admitted.append(e.rid)
            need = [0] * self.cache.n_groups
            for e in entries:
                for g, n in enumerate(self.cache.pages_needed(e.rid, len(e.tokens))):
                    need[g] += n
            for g, n in enumerate(need):
                if n > self.cache.free_pages(g):
                    raise OutOfPages(f"the step needs {n} pages of cache group {g}, {self.cache.free_pages(g)} are free")
            for e in entries:
                assert self.cache.reserve(e.rid, len(e.tokens))
        except OutOfPages:
            for rid in admitted:
                self.cache.release(rid)
            raise

        rids = [e.rid for e in entries]
        q_lens = np.array([len(e.tokens) for e in entries], dtype=np.int32)
        cu = np.zeros(len(entries) + 1, dtype=np.int32)
        np.cumsum(q_lens, out=cu[1:])
        ctx = np.array([self.cache.tokens(r) for r in rids], dtype=np.int32)
        slot = np.array([self.cache.slot(r) for r in rids], dtype=np.int32)
        ids = np.concatenate(token_arrays).astype(np.int32)
        row_req = np.repeat(np.arange(len(entries), dtype=np.int32), q_lens)
        pos = (np.arange(ids.size, dtype=np.int32) - cu[:-1][row_req]) + ctx[row_req]
        logit_rows = np.array([cu[i] + w for i, e in enumerate(entries) for w in e.want], dtype=np.int32)
        tables = [self.cache.block_table(rids, g) for g in range(self.cache.n_groups)]
        self.device_cache.clear_fresh_slots()
        return self._stager.stage(ids, pos.astype(np.int32), row_req, cu, ctx, slot, logit_rows, tables)

    def step(self, entries: Sequence[Entry]) -> Optional[torch.Tensor]:
        """Runs one batch; returns float32 logits [wanted places, vocab] in the order of the
        entries and of their `want` (None if nothing is wanted)."""
        entries = [e if isinstance(e, Entry) else Entry(*e) for e in entries]
        batch = self.prepare(entries)
        logits = self.model.forward(batch, self._views)
        for e in entries:
            self.cache.commit(e.rid, len(e.tokens))
        return logits
