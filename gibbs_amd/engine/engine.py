"""The engine: a model bound to its weights and cache, and the one step function.

`step(entries)` runs exactly the tokens it is given, as one batch, from the cache that earlier
steps left, and returns the logits at the wanted places.  The reference's counterpart is
`NativeLm::forward(tokens, start_pos, state)` for one sequence
(src/model/native.rs:78-83, src/runtime/lm.rs:513-583); here a
step takes any mix of prompt portions and decoded tokens of several requests.  Its guards are
the reference's (lm.rs:528-544): no empty token list, no position beyond the context limit.
"""
from __future__ import annotations

import ctypes
import itertools
import os
from typing import Dict, Hashable, List, Optional, Sequence

import numpy as np
import torch

from ..cache import CacheManager, DeviceCache, host
from ..config import config_from_dict, read_config_json
from ..config.base import ArchConfig
from ..ops.lib import KernelError, library
from ..parts import DecoderModel, Runtime
from ..parts.native import NativePlan
from ..weights import WeightStore, load_weights, table_of
from .batch import BatchStager, Entry, StepBatch

DEFAULT_PAGE_SIZE = 16      # tokens per cache page, the reference's block size (src/kv/mod.rs:6)
DEFAULT_MAX_CONTEXT = 4096  # the context limit when none is asked for, if the model allows as much
DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32}


class OutOfPages(RuntimeError):
    """The step needs more cache pages (or a slot) than are free; nothing was changed."""


class StepError(ValueError):
    """The step's entries cannot be run (empty tokens, bad ids, context limit, unknown request)."""


class Engine:
    def __init__(self, model_dir: Optional[str] = None, *, dtype: str = "bfloat16", max_tokens: int = 8192,
                 max_requests: int = 8, page_size: int = DEFAULT_PAGE_SIZE, device: str = "cuda:0", arch: Optional[str] = None,
                 ctx: Optional[int] = None, config: Optional[ArchConfig] = None,
                 weights: Optional[WeightStore] = None, fold_gains: bool = True, fused_decode_rows: int = 64,
                 group_pages: Optional[Sequence[int]] = None):
        """`model_dir`: a folder with config.json and model.safetensors (the model class is chosen
        by config.json).  `max_tokens`: tokens the cache pool holds (each request's count rounded
        up to whole pages).  `ctx`: context limit, default config.json's max_position_embeddings or 4,096,
        whichever is smaller.
        `config` + `weights` may stand in for a folder (weights already on the device).
        `fold_gains=False` keeps the norms' gains out of the bfloat16 matrices and `fused_decode_rows=0`
        keeps steps of decoded tokens off the fused decode kernels: the same model on the general path,
        for comparisons.  `group_pages`: pages of every cache group's pool, one count per group in
        the order the groups first appear in the layer order (default: `max_tokens` worth for each; a
        group with a window can do with about max_requests x (window + longest portion) tokens)."""
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
        # the reference's default: first(runtime.ctx, min(max_position_embeddings or 2048, 4096)) (arch/families/lfm2.json5:50)
        self.ctx_limit = int(ctx) if ctx else min(self.spec.max_position or 2048, DEFAULT_MAX_CONTEXT)
        num_pages = max(1, -(-max_tokens // page_size))
        self.rt = Runtime(self.device, self.dtype, max_positions=min(self.ctx_limit, num_pages * page_size),
                          fold_gains=fold_gains, fused_decode_rows=fused_decode_rows)
        self.model.bind(weights, self.rt)
        self.weight_bytes = weights.nbytes()
        del weights

        self.cache = CacheManager(self.model.cache_needs(), self.model.state_needs(), page_size,
                                  num_pages if group_pages is None else list(group_pages), max_requests)
        self.device_cache = DeviceCache(self.cache, self.dtype, self.device)
        # the cache views of every run's mixers, by role (a cache owner is a mixer of a run)
        self._views: List[Dict[str, object]] = [{} for _ in self.spec.order]
        for owner, ((run, role), src) in enumerate(zip(self.model.cache_owners(), self.model.kv_sources())):
            self._views[run][role] = self.device_cache.layer_view(owner, src)
        self._stager = BatchStager(self.device)
        self.plan = NativePlan.build(self.model, self._views, self.rt)

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
        """Checks the entries, takes slots and pages for them (all or nothing for the whole step)
        and stages the batch's metadata.  The checks, the page accounting and the packing of the
        staging buffer run in the host runtime (csrc/host/cache_core.cpp)."""
        if not entries:
            raise StepError("a step needs at least one entry")
        cache, lib = self.cache, host.library()
        n = len(entries)
        if len({e.rid for e in entries}) != n:
            twice = next(e.rid for i, e in enumerate(entries) if any(o.rid == e.rid for o in entries[:i]))
            raise StepError(f"request {twice!r} appears twice in one step")
        admitted = []
        try:
            for e in entries:
                if e.rid not in cache:
                    if not cache.admit(e.rid):
                        raise OutOfPages(f"no free slot for request {e.rid!r} ({cache.max_requests} live)")
                    admitted.append(e.rid)
            slots = np.fromiter((cache.slot(e.rid) for e in entries), dtype=np.int32, count=n)
            q_len = np.fromiter((len(e.tokens) for e in entries), dtype=np.int32, count=n)
            try:
                tokens = np.fromiter(itertools.chain.from_iterable(e.tokens for e in entries), dtype=np.int32,
                                     count=int(q_len.sum()))
            except (OverflowError, TypeError, ValueError) as exc:
                raise StepError(f"token ids must be integers that fit 32 bits: {exc}") from None
            want_cu = np.zeros(n + 1, dtype=np.int32)
            np.cumsum([len(e.want) for e in entries], out=want_cu[1:])
            want = np.fromiter(itertools.chain.from_iterable(e.want for e in entries), dtype=np.int32,
                               count=int(want_cu[-1]))
            info = (ctypes.c_long * (1 + cache.n_groups))()
            bad = ctypes.c_int(0)
            operands = (n, slots.ctypes.data, q_len.ctypes.data, tokens.ctypes.data, want_cu.ctypes.data,
                        want.ctypes.data)
            code = lib.gibbs_cache_reserve_step(cache.core, *operands, self.spec.vocab, self.ctx_limit, info,
                                                ctypes.byref(bad))
            if code == host.ERR_NO_ROOM:
                raise OutOfPages(host.last_error())
            if code < 0:
                raise StepError(f"request {entries[bad.value].rid!r}: {host.last_error()}")
        except (OutOfPages, StepError):
            for rid in admitted:
                cache.release(rid)
            raise
        self.device_cache.clear_fresh_slots()
        widths = [int(info[1 + g]) for g in range(cache.n_groups)]
        return self._stager.stage_native(lib, cache.core, operands, info, widths, int(want_cu[-1]))

    def forward(self, batch: StepBatch, workspace: Optional[torch.Tensor] = None, x_in: Optional[torch.Tensor] = None,
                mirror_in: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
        """The model's forward pass over a staged batch: one native call (`workspace`, `x_in`,
        `mirror_in`: see `NativePlan.step`)."""
        return self.plan.step(batch, workspace, x_in, mirror_in)

    def step(self, entries: Sequence[Entry]) -> Optional[torch.Tensor]:
        """Runs one batch; returns float32 logits [wanted places, vocab] in the order of the
        entries and of their `want` (None if nothing is wanted)."""
        entries = [e if isinstance(e, Entry) else Entry(*e) for e in entries]
        batch = self.prepare(entries)
        logits = self.forward(batch)
        for e in entries:
            self.cache.commit(e.rid, len(e.tokens))
        return logits
