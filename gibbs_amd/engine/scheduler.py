"""Continuous batching above the step function.

Policy follows the reference's scheduler (/root/reference/src/scheduler/mod.rs:1128-1580):
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
no request can move at all, the youngest is preempted so that the oldest can.  A request that
does not fit the whole pool alone fails with an error.
"""
from __future__ import annotations

import itertools
from collections import deque
from dataclasses import dataclass, field
from enum import Enum
from typing import Callable, Deque, Dict, Hashable, List, Optional, Tuple
from typing import Sequence as SeqOf

from ..cache.manager import CacheManager
from ..sampling.sampler import Draw, SamplingParams
from .batch import Entry

MAX_PREFILL_CHUNK = 2048            # most prompt tokens one step prefills (scheduler/mod.rs:341)


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


class ContinuousBatchScheduler:
    def __init__(self, cache: CacheManager, runner: Runner, *, context_len: int,
                 max_batch_tokens: int = MAX_PREFILL_CHUNK, chunk: Optional[int] = None,
                 eos_token_ids: SeqOf[int] = ()):
        """`cache`: the engine's cache manager (pages and slots are taken here, before a step
        runs).  `runner`: runs one batch and samples.  `max_batch_tokens`: prompt tokens per step.
        `chunk`: most prompt tokens of one request per step (None: the budget)."""
        if max_batch_tokens < 1 or (chunk is not None and chunk < 1):
            raise ValueError("max_batch_tokens and chunk must be at least 1")
        self.cache = cache
        self.runner = runner
        self.context_len = context_len
        self.max_batch_tokens = max_batch_tokens
        self.chunk = chunk
        self.eos = set(eos_token_ids)
        self.waiting: Deque[Sequence] = deque()
        self.active: List[Sequence] = []
        self.finished: Dict[Hashable, Sequence] = {}
        self._counter = itertools.count()
        self.steps = 0

    # ------------------------------------------------------------------ submitting
    def submit(self, prompt_tokens: SeqOf[int], params: Optional[SamplingParams] = None,
               rid: Optional[Hashable] = None) -> Hashable:
        """Queues a request.  An empty prompt becomes [1] (scheduler/mod.rs:1005-1008);
        `max_new_tokens` is clamped to the room the context leaves (:953-955)."""
        params = params or SamplingParams()
        order = next(self._counter)
        rid = order if rid is None else rid
        if rid in self.finished or any(s.id == rid for s in itertools.chain(self.waiting, self.active)):
            raise KeyError(f"request id {rid!r} is in use")
        prompt = [int(t) for t in prompt_tokens] or [1]
        if len(prompt) > self.context_len:
            raise ValueError(f"the prompt has {len(prompt)} tokens, the context holds {self.context_len}")
        room = self.context_len - len(prompt)
        if params.max_new_tokens > room:
            params = SamplingParams(params.temperature, params.top_p, params.top_k, room, params.seed,
                                    params.ignore_eos)
        self.waiting.append(Sequence(rid, prompt, params, order))
        return rid

    def has_work(self) -> bool:
        return bool(self.waiting or self.active)

    # ------------------------------------------------------------------ helpers
    def _computed(self, seq: Sequence) -> int:
        return self.cache.tokens(seq.id) if seq.id in self.cache else 0

    def _remaining(self, seq: Sequence) -> int:
        """Tokens the request still has to feed: its whole remaining prompt, or 1 when it decodes."""
        return len(seq.prompt_tokens) + len(seq.output_tokens) - self._computed(seq)

    def _fits(self, rid: Hashable, n: int) -> bool:
        need = self.cache.pages_needed(rid, n)
        return all(k <= self.cache.free_pages(g) for g, k in enumerate(need))

    def _largest_fit(self, rid: Hashable, n: int) -> int:
        """The most tokens <= n whose pages are free now (the pages needed grow with n)."""
        lo, hi = 0, n
        while lo < hi:
            mid = (lo + hi + 1) // 2
            if self._fits(rid, mid):
                lo = mid
            else:
                hi = mid - 1
        return lo

    def _finish(self, seq: Sequence, reason: FinishReason, error: Optional[str] = None) -> None:
        seq.state, seq.finish_reason, seq.error = SequenceState.FINISHED, reason, error
        if seq.id in self.cache:
            self.cache.release(seq.id)
        if seq in self.active:
            self.active.remove(seq)
        self.finished[seq.id] = seq

    def _preempt(self, seq: Sequence) -> None:
        """Frees everything the request holds; it will be recomputed from its tokens so far."""
        self.cache.release(seq.id)
        self.active.remove(seq)
        seq.state = SequenceState.WAITING
        seq.preemptions += 1
        self.waiting.appendleft(seq)

    # ------------------------------------------------------------------ one step
    def step(self) -> StepOutput:
        self.steps += 1
        budget = self.max_batch_tokens
        cap = budget if self.chunk is None else min(budget, self.chunk)
        preempted: List[Hashable] = []
        finished: List[Hashable] = []

        # 1. admission: first in, first out; needs a slot and the pages of the first portion
        while self.waiting:
            seq = self.waiting[0]
            if seq.params.max_new_tokens == 0 and not seq.output_tokens:
                self.waiting.popleft()
                self._finish(seq, FinishReason.LENGTH)              # scheduler/mod.rs:1357-1359
                finished.append(seq.id)
                continue
            total = seq.n_tokens
            if self.cache.pages_for(total + 1) > min((p.num_pages for p in self.cache.pools), default=1 << 60):
                self.waiting.popleft()
                self._finish(seq, FinishReason.ERROR,
                             f"the request needs {self.cache.pages_for(total + 1)} pages, the pool has "
                             f"{min(p.num_pages for p in self.cache.pools)}")
                finished.append(seq.id)
                continue
            if not self.cache.admit(seq.id):
                break
            first = min(total, cap)
            if not self.cache.reserve(seq.id, first):
                self.cache.release(seq.id)
                break
            self.waiting.popleft()
            seq.state = SequenceState.PREFILLING
            self.active.append(seq)

        # 2. order: decoders first, then shortest remaining prompt; the oldest prefilling request
        #    keeps up to half the budget
        def is_decoding(s: Sequence) -> bool:
            return s.state == SequenceState.DECODING
        self.active.sort(key=lambda s: (0 if is_decoding(s) else self._remaining(s), s.submitted))
        prefilling = [s for s in self.active if not is_decoding(s)]
        oldest = min(prefilling, key=lambda s: s.submitted, default=None)
        reserved = min(self._remaining(oldest), -(-budget // 2)) if oldest is not None else 0

        # 3. plan: pages first, so that the batch that runs is the batch that fits
        plan: List[Tuple[Sequence, int]] = []
        left = budget
        for seq in list(self.active):
            if seq not in self.active:
                continue                                            # preempted meanwhile
            if is_decoding(seq):
                while not self._fits(seq.id, 1):
                    victim = max(self.active, key=lambda s: s.submitted)
                    plan = [(s, n) for s, n in plan if s is not victim]
                    self._preempt(victim)
                    preempted.append(victim.id)
                    if victim is seq:
                        break
                if seq in self.active:
                    assert self.cache.reserve(seq.id, 1)
                    plan.append((seq, 1))
                continue
            if seq is oldest:
                available, reserved = left, 0
            else:
                available = max(0, left - reserved)
            n = min(self._remaining(seq), available, cap)
            if n > 0 and not self._fits(seq.id, n):
                n = self._largest_fit(seq.id, n)
            if n <= 0:
                continue                                            # budget or pages exhausted: next step
            assert self.cache.reserve(seq.id, n)
            plan.append((seq, n))
            left -= n
        if not plan and self.active:
            # nothing can move: make room for the oldest by preempting the youngest
            victim = max(self.active, key=lambda s: s.submitted)
            if len(self.active) == 1:
                self._finish(victim, FinishReason.ERROR, "the cache pool is too small for this request")
                finished.append(victim.id)
            else:
                self._preempt(victim)
                preempted.append(victim.id)

        # 4. one batch: portions beside decoded tokens; logits at the last row of every request
        #    that has fed all its tokens
        entries: List[Entry] = []
        draws: List[Draw] = []
        sampled_for: List[Sequence] = []
        prefill_tokens = decode_tokens = 0
        for seq, n in plan:
            at = self._computed(seq)
            toks = seq.span(at, n)
            last = at + n == seq.n_tokens
            entries.append(Entry(seq.id, toks, [n - 1] if last else []))
            if last:
                draws.append(Draw(seq.params, seq.id, len(seq.output_tokens)))
                sampled_for.append(seq)
            if is_decoding(seq):
                decode_tokens += 1
            else:
                prefill_tokens += n
        emitted: List[Tuple[Hashable, int]] = []
        if entries:
            try:
                tokens = self.runner(entries, draws)
            except Exception as exc:                                # scheduler/mod.rs:1332-1340
                for seq, _ in plan:
                    self._finish(seq, FinishReason.ERROR, f"{type(exc).__name__}: {exc}")
                    finished.append(seq.id)
                return StepOutput(entries, [], finished, preempted, prefill_tokens, decode_tokens,
                                  len(self.active), len(self.waiting))
            assert len(tokens) == len(sampled_for)
            # 5. emit and finish
            for seq, tok in zip(sampled_for, tokens):
                seq.state = SequenceState.DECODING
                if tok in self.eos and not seq.params.ignore_eos:
                    self._finish(seq, FinishReason.STOP)            # the end token is not emitted
                    finished.append(seq.id)
                    continue
                seq.output_tokens.append(int(tok))
                emitted.append((seq.id, int(tok)))
                if (len(seq.output_tokens) >= seq.params.max_new_tokens
                        or seq.n_tokens >= self.context_len):
                    self._finish(seq, FinishReason.LENGTH)
                    finished.append(seq.id)
        return StepOutput(entries, emitted, finished, preempted, prefill_tokens, decode_tokens,
                          len(self.active), len(self.waiting))

    # ------------------------------------------------------------------ bursts of decode steps
    def burst_plan(self, cap: int) -> Optional[Tuple[List[Sequence], int]]:
        """When nothing waits and every running request decodes, several decode steps may run back to
        back on the device without the host in between (a captured graph per step).  Returns the
        requests (oldest first) and how many steps all of them can still take, at most `cap`; None
        when a step has anything else to do."""
        if self.waiting or not self.active:
            return None
        if any(s.state != SequenceState.DECODING or self._remaining(s) != 1 for s in self.active):
            return None
        seqs = sorted(self.active, key=lambda s: s.submitted)
        n = min(cap, min(min(s.params.max_new_tokens - len(s.output_tokens), self.context_len - s.n_tokens)
                         for s in seqs))
        return (seqs, n) if n >= 1 else None

    def apply_burst(self, seqs: List[Sequence], tokens: List[List[int]]) -> StepOutput:
        """Books the tokens that a burst sampled (tokens[i]: those of seqs[i], all already cached):
        the same emitting and finishing rules as a step, token by token."""
        self.steps += len(tokens[0]) if tokens else 0
        emitted: List[Tuple[Hashable, int]] = []
        finished: List[Hashable] = []
        for seq, toks in zip(seqs, tokens):
            for tok in toks:
                if tok in self.eos and not seq.params.ignore_eos:
                    self._finish(seq, FinishReason.STOP)
                    finished.append(seq.id)
                    break
                seq.output_tokens.append(int(tok))
                emitted.append((seq.id, int(tok)))
                if (len(seq.output_tokens) >= seq.params.max_new_tokens
                        or seq.n_tokens >= self.context_len):
                    self._finish(seq, FinishReason.LENGTH)
                    finished.append(seq.id)
                    break
        return StepOutput([], emitted, finished, [], 0, len(emitted), len(self.active), len(self.waiting))

    def run(self, on_step: Optional[Callable[[StepOutput], None]] = None) -> Dict[Hashable, Sequence]:
        """Steps until every submitted request has finished."""
        while self.has_work():
            out = self.step()
            if on_step is not None:
                on_step(out)
        return self.finished
