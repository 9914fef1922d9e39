"""Generation through the scheduler: the Python entry point and what the command line prints.

`Generator` ties an `Engine` to a `ContinuousBatchScheduler` and a `Sampler`, in the manner of the
reference's one-shot path (src/scheduler/mod.rs:1080-1120,
src/main.rs:741-772): submit, step until done, report prefill and decode speed.
"""
from __future__ import annotations

import time
from dataclasses import dataclass, field
from typing import Callable, Dict, Hashable, List, Optional, Sequence, Union

import torch

from .. import ops
from ..sampling.sampler import Draw, Sampler, SamplingParams
from .batch import Entry
from .decode import DecodeLoop
from .engine import Engine, OutOfPages
from .scheduler import MAX_PREFILL_CHUNK, ContinuousBatchScheduler, FinishReason, StepOutput


@dataclass
class Generation:
    rid: Hashable
    prompt_tokens: List[int]
    tokens: List[int]
    finish_reason: str
    error: Optional[str] = None
    preemptions: int = 0
    ttft_s: Optional[float] = None      # submission to first token (the reference's telemetry keeps the same two
    itl_s: Optional[float] = None       # figures, src/telemetry/mod.rs:228-447); mean time between later tokens


@dataclass
class GenerationStats:
    prefill_tokens: int = 0
    prefill_seconds: float = 0.0
    decode_tokens: int = 0
    decode_seconds: float = 0.0
    steps: int = 0

    @property
    def prefill_tok_s(self) -> float:
        return self.prefill_tokens / max(self.prefill_seconds, 1e-9)

    @property
    def decode_tok_s(self) -> float:
        return self.decode_tokens / max(self.decode_seconds, 1e-9)


# a burst shorter than this does not get a decode loop (and captured graphs) made for it
MIN_STEPS_FOR_NEW_LOOP = 8
# Rows that decode loops are made for: a burst of n requests runs in the loop of the next size up, its other
# rows being padding, so that requests that finish one after another stay on captured graphs all the way down
# instead of having a loop made for every batch size.  The sizes are where the decode step's time steps up
# (its kernels change shape beyond 8, 16, 32 and 48 rows); beyond 64 rows, multiples of 32.
LOOP_ROWS = (1, 2, 4, 8, 16, 32, 48, 64)


def loop_rows(n: int) -> int:
    return next((r for r in LOOP_ROWS if r >= n), -(-n // 32) * 32)


class Generator:
    def __init__(self, engine: Engine, *, max_batch_tokens: Union[int, str] = MAX_PREFILL_CHUNK, chunk: Optional[int] = None,
                 eos_token_ids: Optional[Sequence[int]] = None, decode_burst: int = 16):
        """`max_batch_tokens`: prompt tokens per step, or "auto" for the budget that the scheduler sizes
        by measured costs.  `decode_burst`: while nothing waits and every running request decodes, up to
        this many decode steps run back to back as captured graphs (0: every step goes through the host)."""
        self.engine = engine
        self.decode_burst = decode_burst
        self._loops: Dict[tuple, DecodeLoop] = {}
        self._stepped = True        # a host-driven step ran since the last burst: the loops' device state is stale
        self.sampler = Sampler(engine.device)
        eos = engine.spec.eos_token_ids if eos_token_ids is None else eos_token_ids
        self.scheduler = ContinuousBatchScheduler(engine.cache, self._run, context_len=engine.ctx_limit,
                                                  max_batch_tokens=max_batch_tokens, chunk=chunk, eos_token_ids=eos,
                                                  one_off_work=ops.one_off_work)
        self.stats = GenerationStats()
        self._times: Dict[Hashable, List[float]] = {}       # request -> [submitted, first token, last token, tokens]

    def _run(self, entries: Sequence[Entry], draws: Sequence[Draw]) -> List[int]:
        logits = self.engine.step(entries)
        if logits is None:
            return []
        return self.sampler.sample(logits, draws)

    def submit(self, prompt_tokens: Sequence[int], params: Optional[SamplingParams] = None,
               rid: Optional[Hashable] = None) -> Hashable:
        rid = self.scheduler.submit(prompt_tokens, params, rid)
        self._times[rid] = [time.perf_counter(), 0.0, 0.0, 0]
        return rid

    def _burst(self) -> Optional[StepOutput]:
        plan = self.scheduler.burst_plan(self.decode_burst) if self.decode_burst > 0 else None
        if plan is None:
            return None
        seqs, n, longest = plan
        rids = [s.id for s in seqs]
        params = [s.params for s in seqs]
        greedy = all(p.greedy for p in params)
        if not greedy and not all(not p.greedy for p in params):
            return None                                     # mixed greedy and sampled: step by step
        if any(p.penalises for p in params):
            return None                                     # the penalty reads the recent tokens on the host
        last = [s.output_tokens[-1] for s in seqs]
        index = [len(s.output_tokens) for s in seqs]
        key = (loop_rows(len(seqs)), greedy)
        loop = self._loops.get(key)
        # Requests that reach their token limits one after another would cut every burst at the next one to end.
        # The rows of a loop cost what they cost, live or not: the burst runs until the last of them ends (where the
        # pages allow it), and the tokens behind a request's limit are dropped like those behind an end of sequence.
        spans = [longest, n] if longest > n else [n]
        if loop is None and spans[0] < MIN_STEPS_FOR_NEW_LOOP:
            # capturing graphs for so few steps costs more than it saves; a loop that was made for more rows
            # serves as well, while its step costs less than a step through the host (up to twice the rows)
            loop = next((l for (rows, g), l in sorted(self._loops.items(), key=lambda kv: kv[0][0])
                         if g == greedy and key[0] < rows <= 2 * key[0]), None)
            if loop is None:
                return None
        tokens = None
        for n in spans:
            try:
                if loop is None:
                    loop = self._loops[key] = DecodeLoop(self.engine, rids, last, params, first_index=index, rows=key[0])
                elif self._stepped or loop.rids != rids or loop.steps_done + n > loop.capacity:
                    loop.rebind(rids, last, params, index)
                else:
                    loop.params, loop.index = params, [i - loop.steps_done for i in index]
                self._stepped = False
                started = self.scheduler.clock()
                loop.run(n)
                tokens = loop.tokens(last=n)                # (reading them back waits for the steps)
                break
            except OutOfPages:
                continue                                    # the shorter span; or let the scheduler make room
        if tokens is None:
            return None
        if self.scheduler.tuner is not None:
            self.scheduler.tuner.record((self.scheduler.clock() - started) / n, 0, len(seqs))
        return self.scheduler.apply_burst(seqs, tokens)

    def step(self) -> StepOutput:
        """One scheduler step (or one burst of decode steps), timed: a step that holds prompt tokens
        counts as prefill (with its decoded tokens riding along), any other as decode."""
        torch.cuda.synchronize(self.engine.device)
        t0 = time.perf_counter()
        out = self._burst()
        if out is None:
            out = self.scheduler.step()
            self._stepped = True
        torch.cuda.synchronize(self.engine.device)
        now = time.perf_counter()
        dt = now - t0
        last = t = object()
        for rid, _ in out.emitted:          # (a burst's tokens come request by request)
            if rid is not last and rid != last:
                last, t = rid, self._times.get(rid)
                if t is not None:
                    if t[3] == 0:
                        t[1] = now
                    t[2] = now
            if t is not None:
                t[3] += 1
        self.stats.steps += 1
        if out.prefill_tokens:
            self.stats.prefill_tokens += out.prefill_tokens
            self.stats.prefill_seconds += dt
        elif out.decode_tokens:
            self.stats.decode_tokens += out.decode_tokens
            self.stats.decode_seconds += dt
        return out

    def run(self, on_step: Optional[Callable[[StepOutput], None]] = None) -> Dict[Hashable, Generation]:
        """Steps until every submitted request has finished.  `on_step` sees every step's output as it
        happens (`emitted`: the (request, token) pairs of the step or burst), for callers that stream."""
        while self.scheduler.has_work():
            out = self.step()
            if on_step is not None:
                on_step(out)
        return self.results()

    def results(self) -> Dict[Hashable, Generation]:
        out = {}
        for rid, s in self.scheduler.finished.items():
            t = self._times.get(rid, [0.0, 0.0, 0.0, 0])
            out[rid] = Generation(rid, s.prompt_tokens, list(s.output_tokens),
                                  s.finish_reason.value if s.finish_reason else "stop", s.error, s.preemptions,
                                  ttft_s=t[1] - t[0] if t[3] else None,
                                  itl_s=(t[2] - t[1]) / (t[3] - 1) if t[3] > 1 else None)
        return out


def generate(engine: Engine, prompts: Sequence[Sequence[int]], max_tokens: int = 64,
             temperature: Optional[float] = None, top_p: Optional[float] = None, top_k: int = 50, seed: int = 0,
             ignore_eos: bool = False, max_batch_tokens: Union[int, str] = MAX_PREFILL_CHUNK,
             chunk: Optional[int] = None, decode_burst: int = 16, repetition_penalty: float = 1.0) -> List[Generation]:
    """Generates a continuation of every prompt (lists of token ids), batched continuously."""
    gen = Generator(engine, max_batch_tokens=max_batch_tokens, chunk=chunk, decode_burst=decode_burst)
    params = SamplingParams(temperature, top_p, top_k, max_tokens, seed, ignore_eos, repetition_penalty)
    rids = [gen.submit(p, params) for p in prompts]
    results = gen.run()
    return [results[r] for r in rids]
