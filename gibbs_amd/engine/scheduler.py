"""Continuous batching above the step function.

Policy follows the reference's scheduler (src/scheduler/mod.rs:1128-1580):
  * waiting requests are admitted first-in first-out while a slot and the pages of their first
    portion are free; the first that does not fit goes back to the front and admission stops for
    this step (:1155-1221);
  * a step hands out a budget of prompt tokens, shortest remaining prompt first, while the
    oldest prefilling request keeps up to half the budget reserved for itself (:1235-1246,
    :1271-1283);
  * every decoding request gets exactly one token per step (:1376-1487);
  * a request ends on an end-of-sequence token (not emitted, `stop`), at `max_new_tokens` or at
    the context limit (`length`), or on an error (:1357-1373, :1505-1528); its pages and slot go
    back at once (:1539-1569).
Unlike the reference, which runs each sequence's forward pass on its own, all portions and all
decoded tokens of a step form one batch of the step function.

When pages run out (the reference goes on without them, its block ids being bookkeeping only,
:1296-1299, :1397-1400; real pages cannot): a decoding request that cannot get its next page
takes it from the youngest running request, which is preempted: its pages and slot are freed and
it returns to the front of the waiting queue with all its tokens so far, to be recomputed as a
prompt (state of fixed size cannot be rewound or swapped by position, so recomputation is the
only exact way).  A prompt portion that cannot get pages shrinks to what is free, or waits.  If
no request can move at all, the youngest is preempted so that the oldest can.  Admission leaves,
beside the pages of the newcomer's first portion, the page that every running request needs for
its next token: a preempted request must not take the freed page straight back.  A request that
does not fit the whole pool alone fails with an error.

The decisions themselves are native code (csrc/host/scheduler.cpp: it works on lengths and counts and
takes slots and pages from the cache core directly); this module keeps the tokens, the sampling
parameters and the results, builds the step's entries from the native plan, runs them and reports
the sampled tokens back.
"""
from __future__ import annotations

import ctypes
import dataclasses
import itertools
import time
from collections import deque
from dataclasses import dataclass, field
from enum import Enum
from typing import Callable, Deque, Dict, Hashable, List, Optional, Tuple, Union
from typing import Sequence as SeqOf

from ..cache import host
from ..cache.manager import CacheManager
from ..sampling.sampler import RECENT_TOKENS, Draw, SamplingParams
from .batch import Entry

MAX_PREFILL_CHUNK = 2048            # most prompt tokens one step prefills (scheduler/mod.rs:341)
INITIAL_PREFILL_CHUNK = 64          # the budget before any prefill has been timed (scheduler/mod.rs:345)
IDLE_STEP_SECONDS = 0.1             # with nothing decoding a step's prefill is sized to take this long (:348)


class PrefillTuner:
    """The reference's measured budget of prompt tokens per step (scheduler/mod.rs:359-403): while
    requests decode, a step's prompt tokens are sized to cost about one decode round (at least one
    token, and one token only until a decode round has been timed); with nothing decoding, about
    100 ms; 64 before any prefill has been timed; never more than 2,048.  Costs are moving averages
    (0.75 old + 0.25 new).  The reference times every sequence's pass by itself; here a step is one
    batch, so a step of prompt tokens beside decoded ones counts as prefill for what it took beyond
    a decode round (and as the decode round itself while none has been timed)."""

    def __init__(self):
        self.prefill_s_per_token = 0.0      # 0: not measured yet
        self.decode_round_s = 0.0

    def budget(self, decoding: bool) -> int:
        if self.prefill_s_per_token == 0.0:
            return INITIAL_PREFILL_CHUNK
        if decoding and self.decode_round_s == 0.0:
            return 1
        target = self.decode_round_s if decoding else IDLE_STEP_SECONDS
        return max(1, min(int(target / self.prefill_s_per_token), MAX_PREFILL_CHUNK))

    def record(self, seconds: float, prefill_tokens: int, decode_tokens: int) -> None:
        ewma = lambda old, new: new if old == 0.0 else 0.75 * old + 0.25 * new
        if prefill_tokens > 0 and decode_tokens > 0:
            if self.decode_round_s == 0.0:
                self.decode_round_s = seconds
                return
            seconds = max(seconds - self.decode_round_s, 0.05 * seconds)
            self.prefill_s_per_token = ewma(self.prefill_s_per_token, seconds / prefill_tokens)
        elif prefill_tokens > 0:
            self.prefill_s_per_token = ewma(self.prefill_s_per_token, seconds / prefill_tokens)
        elif decode_tokens > 0:
            self.decode_round_s = ewma(self.decode_round_s, seconds)


class SequenceState(Enum):          # scheduler/mod.rs:327-332
    WAITING = "waiting"
    PREFILLING = "prefilling"
    DECODING = "decoding"
    FINISHED = "finished"


class FinishReason(Enum):           # scheduler/mod.rs:450-458
    STOP = "stop"
    LENGTH = "length"
    ERROR = "error"


@dataclass(eq=False)         # a request is itself: membership tests compare identity, not token lists
class Sequence:
    id: Hashable
    prompt_tokens: List[int]
    params: SamplingParams
    submitted: int                                  # admission order (a counter, not a clock)
    output_tokens: List[int] = field(default_factory=list)
    state: SequenceState = SequenceState.WAITING
    finish_reason: Optional[FinishReason] = None
    error: Optional[str] = None
    preemptions: int = 0

    @property
    def tokens(self) -> List[int]:
        return self.prompt_tokens + self.output_tokens

    @property
    def n_tokens(self) -> int:
        return len(self.prompt_tokens) + len(self.output_tokens)

    def span(self, at: int, n: int) -> List[int]:
        """tokens[at : at + n] without joining the two lists."""
        p = len(self.prompt_tokens)
        if at >= p:
            return self.output_tokens[at - p:at - p + n]
        if at + n <= p:
            return self.prompt_tokens[at:at + n]
        return self.prompt_tokens[at:] + self.output_tokens[:at + n - p]


@dataclass
class StepOutput:
    """What one scheduler step did."""
    entries: List[Entry]
    emitted: List[Tuple[Hashable, int]]             # (request, token) in batch order
    finished: List[Hashable]
    preempted: List[Hashable]
    prefill_tokens: int = 0
    decode_tokens: int = 0
    active: int = 0
    waiting: int = 0


# runner(entries, draws) -> one sampled token per wanted place, in order
Runner = Callable[[SeqOf[Entry], SeqOf[Draw]], List[int]]


# what the native core reports back: (kind, request number, value)
EV_ADMITTED, EV_RELEASED, EV_PREEMPTED, EV_STOP, EV_LENGTH, EV_TOO_LARGE, EV_POOL, EV_STEP_FAILED = range(1, 9)


class ContinuousBatchScheduler:
    def __init__(self, cache: CacheManager, runner: Runner, *, context_len: int,
                 max_batch_tokens: Union[int, str] = MAX_PREFILL_CHUNK, chunk: Optional[int] = None,
                 eos_token_ids: SeqOf[int] = (), clock: Callable[[], float] = time.perf_counter,
                 one_off_work: Callable[[], int] = lambda: 0):
        """`cache`: the engine's cache manager (pages and slots are taken here, before a step
        runs).  `runner`: runs one batch and samples.  `max_batch_tokens`: prompt tokens per step,
        or "auto" for the reference's measured budget (`PrefillTuner`; `clock` gives its seconds).
        `chunk`: most prompt tokens of one request per step (None: the budget).  `one_off_work`: a
        count that grows when a step did set-up work that its like will not do again (the engine's
        `ops.one_off_work`); such a step's time is kept from the measured budget."""
        self.one_off_work = one_off_work
        self.tuner: Optional[PrefillTuner] = None
        self.clock = clock
        if max_batch_tokens == "auto":
            self.tuner, max_batch_tokens = PrefillTuner(), INITIAL_PREFILL_CHUNK
        if not isinstance(max_batch_tokens, int) or max_batch_tokens < 1 or (chunk is not None and chunk < 1):
            raise ValueError("max_batch_tokens (a number or 'auto') and chunk must be at least 1")
        self.cache = cache
        self.runner = runner
        self.context_len = context_len
        self.max_batch_tokens = max_batch_tokens
        self.chunk = chunk
        self.eos = set(eos_token_ids)
        self.finished: Dict[Hashable, Sequence] = {}
        self.steps = 0
        self._lib = host.library()
        self._core = self._lib.gibbs_sched_create(cache.core, context_len, max_batch_tokens, chunk or 0)
        if not self._core:
            raise ValueError("the scheduler core refused its sizes")
        self._seqs: List[Sequence] = []                     # by request number (the order of submission)
        self._ids: Dict[Hashable, int] = {}                 # requests that have not finished
        room = 3 * (8 * cache.max_requests + 64)
        self._events = (ctypes.c_long * room)()
        self._n_events = ctypes.c_long(0)
        self._plan = (ctypes.c_long * (5 * cache.max_requests))()
        self._numbers = (ctypes.c_int * cache.max_requests)()

    def __del__(self):
        if getattr(self, "_core", None):
            self._lib.gibbs_sched_destroy(self._core)
            self._core = None

    # ------------------------------------------------------------------ submitting
    def submit(self, prompt_tokens: SeqOf[int], params: Optional[SamplingParams] = None,
               rid: Optional[Hashable] = None) -> Hashable:
        """Queues a request.  An empty prompt becomes [1] (scheduler/mod.rs:1005-1008);
        `max_new_tokens` is clamped to the room the context leaves (:953-955)."""
        params = params or SamplingParams()
        order = len(self._seqs)
        rid = order if rid is None else rid
        if rid in self.finished or rid in self._ids:
            raise KeyError(f"request id {rid!r} is in use")
        prompt = [int(t) for t in prompt_tokens] or [1]
        if len(prompt) > self.context_len:
            raise ValueError(f"the prompt has {len(prompt)} tokens, the context holds {self.context_len}")
        room = self.context_len - len(prompt)
        if params.max_new_tokens > room:
            params = dataclasses.replace(params, max_new_tokens=room)
        number = self._lib.gibbs_sched_submit(self._core, len(prompt), params.max_new_tokens, int(params.ignore_eos))
        assert number == order
        self._seqs.append(Sequence(rid, prompt, params, order))
        self._ids[rid] = number
        return rid

    # ------------------------------------------------------------------ what the core knows
    def _listed(self, which: int) -> List[Sequence]:
        out = (ctypes.c_int * max(1, len(self._ids)))()
        n = self._lib.gibbs_sched_list(self._core, which, out, len(out))
        return [self._seqs[out[i]] for i in range(n)]

    @property
    def waiting(self) -> Deque[Sequence]:
        """The waiting queue, head first (a copy: the queue itself is the core's)."""
        return deque(self._listed(0))

    @property
    def active(self) -> List[Sequence]:
        return self._listed(1)

    def _counts(self):
        w, a = ctypes.c_int(0), ctypes.c_int(0)
        self._lib.gibbs_sched_counts(self._core, ctypes.byref(w), ctypes.byref(a))
        return w.value, a.value

    def has_work(self) -> bool:
        return any(self._counts())

    def _book(self, error: Optional[str] = None):
        """Applies the core's events of the last call to the requests and to the cache manager's names;
        returns (finished ids, preempted ids) in the order they happened."""
        finished, preempted = [], []
        if 3 * self._n_events.value > len(self._events):          # more happened than the buffer holds: ask again
            self._events = (ctypes.c_long * (3 * self._n_events.value))()
            self._lib.gibbs_sched_events(self._core, self._events, len(self._events))
        ev = self._events
        for i in range(self._n_events.value):
            kind, seq, value = ev[3 * i], self._seqs[ev[3 * i + 1]], ev[3 * i + 2]
            if kind == EV_ADMITTED:
                self.cache.adopt(seq.id, value)
                seq.state = SequenceState.PREFILLING
            elif kind == EV_RELEASED:
                self.cache.forget(seq.id)
            elif kind == EV_PREEMPTED:
                seq.state = SequenceState.WAITING
                seq.preemptions += 1
                preempted.append(seq.id)
            else:
                seq.state = SequenceState.FINISHED
                if kind == EV_STOP:
                    seq.finish_reason = FinishReason.STOP
                elif kind == EV_LENGTH:
                    seq.finish_reason = FinishReason.LENGTH
                else:
                    seq.finish_reason = FinishReason.ERROR
                    pool = min((p.num_pages for p in self.cache.pools), default=0)
                    seq.error = {EV_TOO_LARGE: f"the request needs {value} pages, the pool has {pool}",
                                 EV_POOL: "the cache pool is too small for this request"}.get(kind, error)
                self.finished[seq.id] = seq
                self._ids.pop(seq.id, None)
                finished.append(seq.id)
        return finished, preempted

    # ------------------------------------------------------------------ one step
    def step(self) -> StepOutput:
        self.steps += 1
        lib, n_ev = self._lib, ctypes.byref(self._n_events)
        if self.tuner is not None:
            decoding = any(s.state == SequenceState.DECODING for s in self.active)
            self.max_batch_tokens = self.tuner.budget(decoding)
            lib.gibbs_sched_set_budget(self._core, self.max_batch_tokens)
        n_plan = lib.gibbs_sched_plan(self._core, self._plan, len(self._plan) // 5, self._events, len(self._events), n_ev)
        if n_plan < 0:
            raise RuntimeError(host.last_error())
        finished, preempted = self._book()

        # one batch: portions beside decoded tokens; logits at the last row of every request that has
        # fed all its tokens
        entries: List[Entry] = []
        draws: List[Draw] = []
        sampled_for: List[Sequence] = []
        prefill_tokens = decode_tokens = 0
        for i in range(n_plan):
            number, at, n, last, decoding = self._plan[5 * i:5 * i + 5]
            seq = self._seqs[number]
            entries.append(Entry(seq.id, seq.span(at, n), [n - 1] if last else []))
            if last:
                recent = seq.tokens[-RECENT_TOKENS:] if seq.params.penalises else ()
                draws.append(Draw(seq.params, seq.id, len(seq.output_tokens), recent))
                sampled_for.append(seq)
            if decoding:
                decode_tokens += 1
            else:
                prefill_tokens += n
        emitted: List[Tuple[Hashable, int]] = []
        if entries:
            started, setup = self.clock(), self.one_off_work()
            try:
                tokens = self.runner(entries, draws)
            except Exception as exc:                                # scheduler/mod.rs:1332-1340
                lib.gibbs_sched_fail_plan(self._core, self._events, len(self._events), n_ev)
                finished += self._book(f"{type(exc).__name__}: {exc}")[0]
                waiting, active = self._counts()
                return StepOutput(entries, [], finished, preempted, prefill_tokens, decode_tokens, active, waiting)
            assert len(tokens) == len(sampled_for)
            if self.tuner is not None and self.one_off_work() == setup:      # (a step that did set-up work is no measure)
                self.tuner.record(self.clock() - started, prefill_tokens, decode_tokens)
            # emit and finish
            k = len(tokens)
            numbers = (ctypes.c_int * max(1, k))(*[s.submitted for s in sampled_for])
            is_eos = (ctypes.c_int * max(1, k))(*[int(t in self.eos) for t in tokens])
            took = (ctypes.c_int * max(1, k))()
            if lib.gibbs_sched_apply(self._core, k, numbers, is_eos, took, self._events, len(self._events), n_ev) < 0:
                raise RuntimeError(host.last_error())
            for seq, tok, counts in zip(sampled_for, tokens, took):
                seq.state = SequenceState.DECODING
                if counts:
                    seq.output_tokens.append(int(tok))
                    emitted.append((seq.id, int(tok)))
            finished += self._book()[0]
        waiting, active = self._counts()
        return StepOutput(entries, emitted, finished, preempted, prefill_tokens, decode_tokens, active, waiting)

    # ------------------------------------------------------------------ bursts of decode steps
    def burst_plan(self, cap: int) -> Optional[Tuple[List[Sequence], int, int]]:
        """When nothing waits and every running request decodes, several decode steps may run back to
        back on the device without the host in between (a captured graph per step).  Returns the
        requests (oldest first), how many steps all of them can still take, at most `cap`, and how many
        steps it is until the last of them reaches its token limit (at most `cap`; a burst may run that
        long: `apply_burst` drops what a request samples beyond its limit); None when a step has anything
        else to do."""
        n_out, longest = ctypes.c_int(0), ctypes.c_long(0)
        n = self._lib.gibbs_sched_burst_plan(self._core, cap, self._numbers, len(self._numbers), ctypes.byref(n_out),
                                             ctypes.byref(longest))
        if n < 1:
            return None
        return [self._seqs[self._numbers[i]] for i in range(n_out.value)], int(n), int(longest.value)

    def apply_burst(self, seqs: List[Sequence], tokens: List[List[int]]) -> StepOutput:
        """Books the tokens that a burst sampled (tokens[i]: those of seqs[i], all already cached):
        the same emitting and finishing rules as a step, token by token (one call of the core for all of them)."""
        k, n = len(seqs), len(tokens[0]) if tokens else 0
        self.steps += n
        flat = (ctypes.c_int * max(1, k * n))(*[t for toks in tokens for t in toks])
        took = (ctypes.c_int * max(1, k))()
        if self._lib.gibbs_sched_apply_burst(self._core, k, host.ints([s.submitted for s in seqs]), n, flat,
                                             host.ints(sorted(self.eos)), len(self.eos), took, self._events,
                                             len(self._events), ctypes.byref(self._n_events)) < 0:
            raise RuntimeError(host.last_error())
        emitted: List[Tuple[Hashable, int]] = []
        for seq, toks, t in zip(seqs, tokens, took):
            mine = toks[:t]
            seq.output_tokens.extend(mine)
            emitted.extend(zip(itertools.repeat(seq.id), mine))
        finished = self._book()[0]
        waiting, active = self._counts()
        return StepOutput([], emitted, finished, [], 0, len(emitted), active, waiting)

    def run(self, on_step: Optional[Callable[[StepOutput], None]] = None) -> Dict[Hashable, Sequence]:
        """Steps until every submitted request has finished."""
        while self.has_work():
            out = self.step()
            if on_step is not None:
                on_step(out)
        return self.finished
