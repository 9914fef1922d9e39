"""The ragged batch of one step: what every kernel reads to find its rows' requests,
positions, pages and state slots.

Request r of the batch brings q_len[r] >= 1 new tokens at positions ctx[r] .. ctx[r] + q_len[r] - 1,
as rows cu[r] .. cu[r+1] of every activation.  Prompt portions (q_len > 1) and decoded tokens
(q_len = 1) mix freely.  All integer metadata travels to the device in one copy.
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass, field
from typing import Hashable, List, Optional, Sequence

import numpy as np
import torch


@dataclass
class Entry:
    """One request's share of a step: its next tokens, and the places among them (0-based)
    whose logits are wanted."""
    rid: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()


@dataclass
class StepBatch:
    n_rows: int
    n_req: int
    n_logits: int
    ids: torch.Tensor            # [N] token ids
    pos: torch.Tensor            # [N] absolute position of each row
    row_req: torch.Tensor        # [N] index of each row's request in this batch
    cu: torch.Tensor             # [R+1] first row of each request
    ctx: torch.Tensor            # [R] positions cached before this step
    slot: torch.Tensor           # [R] state slot of each request
    logit_rows: torch.Tensor     # [M] rows whose logits are wanted
    tables: List[torch.Tensor]   # per cache group: [R, width] page ids
    # host copies, for parts written without a kernel of their own
    q_lens: List[int] = field(default_factory=list)
    ctx_lens: List[int] = field(default_factory=list)
    slots: List[int] = field(default_factory=list)
    max_q: int = 0
    max_seq: int = 0
    lead_single: int = 0         # requests at the head of the batch that bring one token each (decoded tokens)
    decode_graph: bool = False   # metadata lives in static buffers that a captured graph replays over


def leading_single(q_lens: Sequence[int]) -> int:
    n = 0
    for q in q_lens:
        if q != 1:
            break
        n += 1
    return n


class BatchStager:
    """Packs a step's metadata into one pinned buffer and copies it to the device once.
    A small ring of staging buffers, each guarded by an event, lets the host go on while a
    copy is still queued."""

    RING = 4

    def __init__(self, device: torch.device):
        self.device = device
        self._host = [None] * self.RING
        self._events = [None] * self.RING
        self._turn = 0
        self._dev = [None] * self.RING

    def _buffers(self, n: int):
        i = self._turn
        self._turn = (self._turn + 1) % self.RING
        if self._events[i] is not None:
            self._events[i].synchronize()
        if self._host[i] is None or self._host[i].numel() < n:
            cap = max(4096, 1 << (n - 1).bit_length())
            self._host[i] = torch.empty(cap, dtype=torch.int32, pin_memory=True)
            self._dev[i] = torch.empty(cap, dtype=torch.int32, device=self.device)
        return i, self._host[i], self._dev[i]

    def stage_native(self, lib, core, operands, info, widths: Sequence[int], n_logits: int) -> StepBatch:
        """The host runtime packs the step (entries as `operands` of `gibbs_cache_fill_step`, sizes as
        `info` from its reservation) straight into the pinned buffer; one copy takes it to the device."""
        n, slots_ptr, q_len_ptr = operands[0], operands[1], operands[2]
        total = int(info[0])
        i, host_buf, dev = self._buffers(total)
        offsets = (ctypes.c_long * (9 + len(widths)))()
        if lib.gibbs_cache_fill_step(core, *operands, info, host_buf.data_ptr(), offsets) < 0:
            raise RuntimeError(lib.gibbs_host_last_error().decode(errors="replace"))
        dev[:total].copy_(host_buf[:total], non_blocking=True)
        ev = torch.cuda.Event()
        ev.record()
        self._events[i] = ev
        view = host_buf.numpy()
        q_lens = np.ctypeslib.as_array(ctypes.cast(q_len_ptr, ctypes.POINTER(ctypes.c_int)), (n,)).tolist()
        rows = sum(q_lens)
        sizes = [rows, rows, rows, n + 1, n, n, n_logits] + [n * w for w in widths]
        sec = [dev[int(o):int(o) + size] for o, size in zip(offsets, sizes)]
        return StepBatch(
            n_rows=rows, n_req=n, n_logits=n_logits,
            ids=sec[0], pos=sec[1], row_req=sec[2], cu=sec[3], ctx=sec[4], slot=sec[5], logit_rows=sec[6],
            tables=[t.view(n, w) for t, w in zip(sec[7:], widths)],
            q_lens=q_lens, ctx_lens=view[int(offsets[4]):int(offsets[4]) + n].tolist(),
            slots=view[int(offsets[5]):int(offsets[5]) + n].tolist(),
            max_q=int(offsets[7 + len(widths)]), max_seq=int(offsets[8 + len(widths)]),
            lead_single=leading_single(q_lens))

    def stage(self, ids: np.ndarray, pos: np.ndarray, row_req: np.ndarray, cu: np.ndarray, ctx: np.ndarray,
              slot: np.ndarray, logit_rows: np.ndarray, tables: Sequence[np.ndarray]) -> StepBatch:
        parts = [ids, pos, row_req, cu, ctx, slot, logit_rows, *[t.reshape(-1) for t in tables]]
        # every section starts on a 16-byte boundary
        offs, total = [], 0
        for p in parts:
            offs.append(total)
            total += (p.size + 3) // 4 * 4
        i, host, dev = self._buffers(max(total, 4))
        view = host.numpy()
        for o, p in zip(offs, parts):
            view[o:o + p.size] = p
        dev[:total].copy_(host[:total], non_blocking=True)
        ev = torch.cuda.Event()
        ev.record()
        self._events[i] = ev
        sec = [dev[o:o + p.size] for o, p in zip(offs, parts)]
        n_req = ctx.size
        q_lens = np.diff(cu)
        return StepBatch(
            n_rows=int(ids.size), n_req=int(n_req), n_logits=int(logit_rows.size),
            ids=sec[0], pos=sec[1], row_req=sec[2], cu=sec[3], ctx=sec[4], slot=sec[5], logit_rows=sec[6],
            tables=[s.view(t.shape) for s, t in zip(sec[7:], tables)],
            q_lens=q_lens.tolist(), ctx_lens=ctx.tolist(), slots=slot.tolist(),
            max_q=int(q_lens.max()) if n_req else 0, max_seq=int((ctx + q_lens).max()) if n_req else 0,
            lead_single=leading_single(q_lens.tolist()))
