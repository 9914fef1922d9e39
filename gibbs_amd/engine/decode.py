"""Steady decoding of a fixed set of live requests: one token per request per step, sampled on the
device and fed back on the device, the whole step replayed as one captured HIP graph.

The step is the engine's own: the native step (`NativePlan.step`) over a `StepBatch` whose metadata lives in
static device buffers.  What changes between steps (positions, cached lengths, the sampled ids, the random
draws) is updated by a kernel at the end of the step, so a replay needs no host work; pages for all
steps of a `run` are reserved, and the block tables uploaded, before the first of them.  That same
kernel also writes the sampled tokens' embeddings as the next step's residual rows, so a step is: layers,
final norm, head, and one kernel for argmax, log, advance and embedding.
"""
from __future__ import annotations

import contextlib
import gc
from typing import Hashable, List, Optional, Sequence

import numpy as np
import torch

from .. import ops
from ..sampling.rng import request_key, uniform
from ..sampling.sampler import SamplingParams
from .batch import StepBatch
from .engine import Engine, OutOfPages, StepError


# steps per launch of the longer captured graph (a launch costs the host and the queue about as much
# as four kernels of a step)
UNROLL = 8


@contextlib.contextmanager
def capture(graph: "torch.cuda.CUDAGraph"):
    """Captures into `graph` with Python's cycle collector switched off.  The collector may run at
    any allocation; if it then destroys the graphs of a loop that was dropped earlier (a loop, its
    engine and its batch hold each other), a capturing stream refuses the call and the error, raised
    from a destructor, ends the process.  Such garbage waits for the next collection outside a capture
    (collecting it here first would cost tens of milliseconds per capture on a large heap)."""
    was_enabled = gc.isenabled()
    gc.disable()
    try:
        with torch.cuda.graph(graph):
            yield
    finally:
        if was_enabled:
            gc.enable()


class DecodeLoop:
    def __init__(self, engine: Engine, rids: Sequence[Hashable], last_tokens: Sequence[int],
                 params: Optional[Sequence[SamplingParams]] = None, use_graph: bool = True,
                 max_steps: int = 2048, first_index: Optional[Sequence[int]] = None, rows: Optional[int] = None):
        """`rids`: live requests whose prompts are cached; `last_tokens`: the token each one feeds
        next (sampled from its last logits).  `params`: per-request sampling (default greedy);
        `first_index`: for sampled requests, the output index of their next token (for the draws).
        `rows`: make the loop (its static buffers and captured graphs) for this many rows, of which
        the requests take the first: the others are padding that stands for no request (it reads and
        writes the cache's scratch page and slot, and nothing of it is logged), so that one loop serves
        every number of live requests up to `rows` (the reference's decode needs no set-up per batch
        size either, src/scheduler/mod.rs:1376-1487)."""
        self.engine = engine
        if len(rids) == 0:
            raise StepError("a decode loop needs at least one request")
        self.padded = rows is not None
        self.n = max(int(rows or 0), len(rids))
        self.use_graph = use_graph
        self.capacity = max_steps
        self.graph: Optional[torch.cuda.CUDAGraph] = None          # one step
        self.graph_many: Optional[torch.cuda.CUDAGraph] = None     # UNROLL steps: fewer launches from the host
        self._prepared = None                                      # (steps done, steps) that `prepare` last made ready
        self._workspace: Optional[torch.Tensor] = None             # activations of the native step under the captured graphs
        self._allocate(params)
        self.rebind(rids, last_tokens, params, first_index)

    def _allocate(self, params) -> None:
        """Static device buffers of a loop for `n` requests; the captured graph replays over them."""
        engine, b = self.engine, self.n
        cm, dev = engine.cache, engine.device
        self.greedy = params is None or all(p.greedy for p in params)
        # A block table has one entry per logical page (entries of pages that a window has passed stay, as
        # NO_PAGE), so its width follows the context limit; only a group without a window can never name
        # more logical pages than its pool has.
        self.width = [cm.pages_for(engine.ctx_limit) if cm.group_needs[g].window
                      else min(cm.pages_for(engine.ctx_limit), cm.pools[g].num_pages) for g in range(cm.n_groups)]
        # static metadata: ids pos row_req cu ctx slot logit_rows tables...
        sizes = [b, b, b, b + 1, b, b, b] + [b * w for w in self.width]
        offs = np.concatenate([[0], np.cumsum([(s + 3) // 4 * 4 for s in sizes])])
        self._host = np.zeros(int(offs[-1]), dtype=np.int32)
        self._dev = torch.zeros(int(offs[-1]), dtype=torch.int32, device=dev)
        self._sec = [slice(int(offs[i]), int(offs[i]) + sizes[i]) for i in range(len(sizes))]
        d = self._dev
        self.batch = StepBatch(
            n_rows=b, n_req=b, n_logits=b, ids=d[self._sec[0]], pos=d[self._sec[1]], row_req=d[self._sec[2]],
            cu=d[self._sec[3]], ctx=d[self._sec[4]], slot=d[self._sec[5]], logit_rows=d[self._sec[6]],
            tables=[d[self._sec[7 + g]].view(b, w) for g, w in enumerate(self.width)],
            q_lens=[1] * b, ctx_lens=[0] * b, slots=[0] * b, max_q=1, max_seq=0, lead_single=b, decode_graph=True)
        self.log = torch.zeros((self.capacity, b), dtype=torch.int32, device=dev)
        self.counter = torch.zeros(b, dtype=torch.int32, device=dev)          # steps done, per row
        self.live_mask = torch.zeros(b, dtype=torch.int32, device=dev) if self.padded else None   # 0: a row of padding
        # native step: the rows of the residual stream (and their bfloat16 mirror) live here from one step to
        # the next; the end of a step writes the next tokens' embeddings into them
        hidden = engine.spec.hidden
        self.x = torch.zeros((b, hidden), dtype=torch.float32, device=dev)
        self.mirror = torch.zeros((b, hidden), dtype=torch.bfloat16, device=dev) if engine.dtype == torch.bfloat16 else None
        if not self.greedy:
            self.temperature = torch.zeros(b, dtype=torch.float32, device=dev)
            self.top_p = torch.zeros(b, dtype=torch.float32, device=dev)
            self.top_k = torch.zeros(b, dtype=torch.int32, device=dev)
            self.u_all = torch.zeros((self.capacity, b), dtype=torch.float32, device=dev)
            self.u = torch.zeros(b, dtype=torch.float32, device=dev)

    def rebind(self, rids: Sequence[Hashable], last_tokens: Sequence[int],
               params: Optional[Sequence[SamplingParams]] = None, first_index: Optional[Sequence[int]] = None) -> None:
        """Points the loop (and its captured graph, which only knows the static buffers) at another
        set of live requests: as many as the loop was made for, or, for a padded loop, at most as many
        (the rows behind them become padding); greedy loops take greedy requests only."""
        engine, b = self.engine, self.n
        cm = engine.cache
        k = len(rids)
        if len(last_tokens) != k or k == 0 or k > b or (k != b and not self.padded):
            raise StepError(f"this decode loop was made for {'up to ' if self.padded else ''}{b} requests with one last token each")
        for rid in rids:
            if rid not in cm:
                raise StepError(f"request {rid!r} is not live")
        self.rids = list(rids)
        self.params = list(params) if params is not None else [SamplingParams(temperature=0.0)] * k
        if self.greedy != all(p.greedy for p in self.params):
            raise StepError("a decode loop is captured either for greedy or for sampled requests")
        if any(p.penalises for p in self.params):
            raise StepError("a repetition penalty reads the recent tokens on the host: such requests step through the scheduler")
        self.index = list(first_index) if first_index is not None else [0] * k
        h = self._host
        # (rows of padding: token 0 at position 0 with nothing cached, in the scratch slot and page)
        pad = lambda values, fill: np.concatenate([np.asarray(values, dtype=np.int32), np.full(b - k, fill, dtype=np.int32)])
        h[self._sec[0]] = pad(last_tokens, 0)
        lens = pad([cm.tokens(r) for r in self.rids], 0)
        h[self._sec[1]] = lens
        h[self._sec[2]] = np.arange(b)
        h[self._sec[3]] = np.arange(b + 1)
        h[self._sec[4]] = lens
        h[self._sec[5]] = pad([cm.slot(r) for r in self.rids], engine.device_cache.scratch_slot)
        h[self._sec[6]] = np.arange(b)
        self._fill_tables()
        self._dev.copy_(torch.from_numpy(h))
        if self.padded:
            self.live_mask.copy_(torch.from_numpy(pad([1] * k, 0)))
        self.batch.ctx_lens, self.batch.slots = lens.tolist(), h[self._sec[5]].tolist()
        # The longest sequence the loop can reach before it is bound again: kernels choose their key
        # slices by it, and a captured graph keeps that choice, so graphs captured for a shorter bound
        # are dropped.  Powers of two, so that requests that grow do not have graphs captured often.
        reach = min(engine.ctx_limit, int(lens.max()) + self.capacity)
        if reach > self.batch.max_seq:
            self.batch.max_seq = min(engine.ctx_limit, 1 << max(reach - 1, 1).bit_length())
            self.graph = self.graph_many = None
        self.counter.zero_()
        self.steps_done = 0
        self.pending = 0
        self._prepared = None
        self._embed()
        if not self.greedy:
            fill = [1.0] * (b - k)
            self.temperature.copy_(torch.tensor([p.resolved_temperature for p in self.params] + fill, dtype=torch.float32))
            self.top_p.copy_(torch.tensor([p.resolved_top_p for p in self.params] + fill, dtype=torch.float32))
            self.top_k.copy_(torch.tensor([p.top_k for p in self.params] + [1] * (b - k), dtype=torch.int32))

    def _embed(self) -> None:
        """The embeddings of the tokens in `ids` into the loop's residual rows (the first step after binding;
        every later step finds what the end of the step before it wrote)."""
        ops.embed(self.engine.model.table, self.batch.ids, self.n, out=self.x, mirror=self.mirror)

    # ------------------------------------------------------------------ host side
    def _fill_tables(self) -> None:
        cm, k = self.engine.cache, len(self.rids)
        for g, w in enumerate(self.width):
            table = np.full((self.n, w), self.engine.device_cache.scratch_page[g], dtype=np.int32)   # (padding: every position there)
            table[:k] = cm.block_table(self.rids, g, w)
            self._host[self._sec[7 + g]] = table.reshape(-1)

    def _reserve(self, n_steps: int) -> None:
        cm = self.engine.cache
        try:
            grew = cm.reserve_all(self.rids, self.pending + n_steps, self.engine.ctx_limit)
        except ValueError as e:
            raise StepError(str(e)) from None
        if grew is None:
            need = cm.pages_needed_all
            g = next(g for g, k in enumerate(need) if k > cm.free_pages(g))
            raise OutOfPages(f"{n_steps} decode steps need {need[g]} pages of cache group {g}, {cm.free_pages(g)} are free")
        if grew:
            self._fill_tables()
            for g in range(cm.n_groups):
                s = self._sec[7 + g]
                self._dev[s].copy_(torch.from_numpy(self._host[s]))

    pending = 0         # steps run on the device whose tokens the cache manager has not counted yet

    # ------------------------------------------------------------------ one step on the device
    def _step(self) -> None:
        b = self.batch
        logits = self.engine.forward(b, self._workspace, self.x, self.mirror)
        table = self.engine.model.table
        if self.greedy:
            ops.decode_tail(logits, b.ids, b.pos, b.ctx, self.log, self.counter, None, None, self.n, table, self.x, self.mirror,
                            self.live_mask)
        else:
            ops.sample(logits, self.temperature, self.top_p, self.top_k, self.u, out=b.ids)
            ops.decode_tail(None, b.ids, b.pos, b.ctx, self.log, self.counter, self.u, self.u_all, self.n, table, self.x,
                            self.mirror, self.live_mask)

    def prepare(self, n_steps: int) -> None:
        """Everything a `run(n_steps)` needs before its first replay, so that a caller who times
        the run times replays only: pages for the steps are reserved and the tables uploaded, and
        the captured graphs the run will replay exist (capturing runs nothing)."""
        if self._prepared == (self.steps_done, n_steps):
            return
        if self.steps_done + n_steps > self.capacity:
            raise StepError(f"the decode loop was made for {self.capacity} steps")
        self._reserve(n_steps)
        self._draws(n_steps)
        if self.use_graph:
            self._capture(many=n_steps >= UNROLL)
        self._prepared = (self.steps_done, n_steps)

    def _draws(self, n_steps: int) -> None:
        if self.greedy:
            return
        rows = np.array([[uniform(p.seed, request_key(r), self.index[i] + self.steps_done + s)
                          for i, (r, p) in enumerate(zip(self.rids, self.params))] + [0.5] * (self.n - len(self.rids))
                         for s in range(n_steps)], dtype=np.float32)
        self.u_all[self.steps_done:self.steps_done + n_steps].copy_(torch.from_numpy(rows))
        self.u.copy_(self.u_all[self.steps_done])

    def _capture(self, many: bool) -> None:
        if self.graph is None:
            # the native step's activations: a buffer of the loop's own, which the captured graphs replay
            # over (the engine's own may be replaced by a larger one when another step needs more)
            need = self.engine.plan.workspace_bytes(self.batch, self.x, self.mirror)
            if self._workspace is None or self._workspace.numel() < need:
                self._workspace = torch.empty(need, dtype=torch.uint8, device=self.engine.device)
        if self.graph is None:
            # warm up outside capture (lazy initialisation inside libraries), then capture one step
            # (the warm-up step is undone: metadata and per-request state are put back; its key and
            # value writes are rewritten with the same values by the first replay)
            arena = self.engine.device_cache.arena
            state = self._dev.clone(), self.counter.clone(), self.log.clone(), arena.clone()
            self._step()
            torch.cuda.synchronize()
            self._dev.copy_(state[0]); self.counter.copy_(state[1]); self.log.copy_(state[2]); arena.copy_(state[3])
            self._embed()
            if not self.greedy:
                self.u.copy_(self.u_all[self.steps_done])
            g = torch.cuda.CUDAGraph()
            torch.cuda.synchronize()
            with capture(g):
                self._step()
            self.graph = g                                  # the capture itself ran nothing
        if many and self.graph_many is None:
            g = torch.cuda.CUDAGraph()
            torch.cuda.synchronize()
            with capture(g):
                for _ in range(UNROLL):
                    self._step()
            self.graph_many = g

    def run(self, n_steps: int) -> None:
        """Runs `n_steps` decode steps; tokens collect on the device (see `tokens`)."""
        self.prepare(n_steps)
        left = n_steps
        if self.graph_many is not None:
            while left >= UNROLL:
                self.graph_many.replay()
                left -= UNROLL
        for _ in range(left):
            if self.graph is not None:
                self.graph.replay()
            else:
                self._step()
        self.pending += n_steps
        self.steps_done += n_steps
        self._prepared = None
        self.sync_cache()

    def sync_cache(self) -> None:
        """Tells the cache manager about the positions the device has filled."""
        self.engine.cache.commit_all(self.rids, self.pending)
        self.pending = 0

    def tokens(self, last: Optional[int] = None) -> List[List[int]]:
        """Tokens sampled since the loop was bound (or only by the last `last` steps), per request
        (row s of the log is what step s sampled)."""
        first = 0 if last is None else self.steps_done - last
        return self.log[first:self.steps_done, :len(self.rids)].cpu().numpy().T.tolist()
