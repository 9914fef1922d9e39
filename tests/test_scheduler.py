"""The scheduler's decisions, with a fake step function (no GPU).  The policy tests follow the
reference's (src/scheduler/mod.rs:1635-1737, :1873-1931); what happens when pages
run out is this engine's own decision."""
import pytest

from gibbs_amd.cache import CacheManager, CacheNeed, StateNeed
from gibbs_amd.engine.scheduler import ContinuousBatchScheduler, FinishReason, SequenceState
from gibbs_amd.sampling import SamplingParams


class FakeModel:
    """Commits what it is given and 'samples' a function of the request's fed tokens, so that a
    request recomputed after preemption must continue exactly as before."""

    def __init__(self, cache, eos=None):
        self.cache, self.eos, self.batches, self.fed = cache, eos, [], {}

    def __call__(self, entries, draws):
        self.batches.append([(e.rid, len(e.tokens), bool(e.want)) for e in entries])
        out = []
        for e in entries:
            assert e.rid in self.cache, "the scheduler admits before it runs"
            at = self.cache.tokens(e.rid)
            self.fed.setdefault(e.rid, [])
            del self.fed[e.rid][at:]                     # a recomputed request starts over
            assert len(self.fed[e.rid]) == at, "tokens must arrive in order, none twice, none skipped"
            self.fed[e.rid].extend(e.tokens)
            self.cache.commit(e.rid, len(e.tokens))
            if e.want:
                assert list(e.want) == [len(e.tokens) - 1]
                out.append((sum(self.fed[e.rid]) * 31 + len(self.fed[e.rid])) % 1000 + 3)
        assert len(out) == len(draws)
        return out


def make(pages=64, reqs=8, ps=16, budget=64, chunk=None, ctx=4096, eos=()):
    cache = CacheManager([CacheNeed(1, 16), None], [(), (StateNeed("s", (2,)),)], ps, pages, reqs)
    model = FakeModel(cache)
    return ContinuousBatchScheduler(cache, model, context_len=ctx, max_batch_tokens=budget, chunk=chunk,
                                    eos_token_ids=eos), model, cache


def greedy(n):
    return SamplingParams(temperature=0.0, max_new_tokens=n)


def test_one_request_runs_to_max_new_tokens():
    s, model, cache = make()
    rid = s.submit(list(range(10, 30)), greedy(5))
    done = s.run()
    assert done[rid].finish_reason == FinishReason.LENGTH and len(done[rid].output_tokens) == 5
    assert model.batches[0] == [(rid, 20, True)] and all(b == [(rid, 1, True)] for b in model.batches[1:])
    assert len(model.batches) == 5          # the first token comes from the prompt's last logits
    assert cache.free_pages() == 64 and cache.free_slots() == 8
    cache.check()


def test_budget_chunks_and_decoders_never_starve():
    s, model, _ = make(budget=16)
    a = s.submit([1] * 8, greedy(50))
    s.step(); s.step()
    b = s.submit([2] * 100, greedy(2))
    outs = [s.step() for _ in range(8)]
    for o in outs[:6]:
        sizes = {e.rid: len(e.tokens) for e in o.entries}
        assert sizes[a] == 1, "a decoding request gets its token in every step"
        assert sizes.get(b, 0) <= 16
    assert sum(len(e.tokens) for o in outs for e in o.entries if e.rid == b) >= 100


def test_short_prompt_not_stuck_behind_long_and_long_not_starved():
    s, model, _ = make(budget=32)
    long = s.submit([1] * 200, greedy(1))
    s.step()
    short = s.submit([2] * 6, greedy(1))
    o = s.step()
    sizes = {e.rid: len(e.tokens) for e in o.entries}
    assert sizes[short] == 6, "the short prompt is served whole at once"
    assert sizes[long] >= 16, "the oldest prefilling request keeps half the budget"
    # a stream of short prompts cannot hold the long one back
    for i in range(20):
        s.submit([3] * 20, greedy(1))
        s.step()
    assert long in s.finished


def test_chunk_cap_and_wanted_rows():
    s, model, _ = make(budget=64, chunk=8)
    rid = s.submit([1] * 20, greedy(1))
    s.run()
    assert model.batches == [[(rid, 8, False)], [(rid, 8, False)], [(rid, 4, True)]]


def test_finish_reasons():
    s, model, _ = make(eos=(7,))
    model_tokens = iter([5, 7, 9])
    s.runner = lambda entries, draws: [model.__call__(entries, draws) and next(model_tokens)][0:len(draws)]
    rid = s.submit([1, 2, 3], greedy(10))
    done = s.run()
    assert done[rid].finish_reason == FinishReason.STOP and done[rid].output_tokens == [5], "the end token is not emitted"
    s, model, _ = make(eos=(7,))
    rid0 = s.submit([1], greedy(0))
    assert s.run()[rid0].finish_reason == FinishReason.LENGTH and not model.batches
    s, model, _ = make(ctx=12)
    rid = s.submit([1] * 10, greedy(50))
    done = s.run()
    assert done[rid].finish_reason == FinishReason.LENGTH and len(done[rid].output_tokens) == 2, "stops at the context length"
    with pytest.raises(ValueError, match="context holds"):
        s.submit([1] * 13, greedy(1))
    s, model, _ = make()
    assert s.submit([], greedy(1)) in (0,) and s.waiting[0].prompt_tokens == [1]      # an empty prompt becomes [1]


def test_ignore_eos_and_error_path():
    s, model, cache = make(eos=(7,))
    s.runner = lambda entries, draws: [model.__call__(entries, draws) and 7][0:len(draws)]
    rid = s.submit([1, 2], SamplingParams(temperature=0.0, max_new_tokens=3, ignore_eos=True))
    assert s.run()[rid].output_tokens == [7, 7, 7]

    def boom(entries, draws):
        raise RuntimeError("kernel fault")
    s, model, cache = make()
    s.runner = boom
    rid = s.submit([1, 2], greedy(3))
    done = s.run()
    assert done[rid].finish_reason == FinishReason.ERROR and "kernel fault" in done[rid].error
    assert cache.free_pages() == 64 and cache.free_slots() == 8, "a failed request frees what it held"


def test_admission_waits_for_slots_and_pages():
    s, model, cache = make(pages=4, reqs=2, budget=64)
    a = s.submit([1] * 30, greedy(40))       # 2 pages now, grows to 5 > pool? no: 30 + 40 = 70 tokens = 5 pages
    b = s.submit([2] * 30, greedy(2))
    c = s.submit([3] * 10, greedy(2))
    o = s.step()
    assert {e.rid for e in o.entries} == {a, b} and o.waiting == 1, "the third request waits for a slot"
    assert [q.id for q in s.waiting] == [c]
    s.run()
    assert all(r in s.finished for r in (a, b, c))
    cache.check()


def test_pages_run_out_preempts_youngest_and_recomputes():
    # pool of 6 pages of 4 tokens: two requests that grow until they collide
    s, model, cache = make(pages=6, reqs=4, ps=4, budget=64)
    old = s.submit([1] * 8, greedy(12))      # 8 + 12 = 20 tokens = 5 pages
    young = s.submit([2] * 8, greedy(6))     # 8 + 6 = 14 tokens = 4 pages
    preempted = []
    while s.has_work():
        o = s.step()
        preempted += o.preempted
        cache.check()
    assert preempted and set(preempted) == {young}, "the youngest running request is the one preempted"
    done = s.finished
    assert done[old].finish_reason == done[young].finish_reason == FinishReason.LENGTH
    assert len(done[old].output_tokens) == 12 and len(done[young].output_tokens) == 6
    assert done[young].preemptions >= 1 and done[old].preemptions == 0
    # the same requests alone (no pressure) give the same tokens: recomputation is exact
    for rid, prompt, n in ((old, [1] * 8, 12), (young, [2] * 8, 6)):
        s2, _, _ = make(pages=64, ps=4)
        r2 = s2.submit(prompt, greedy(n))
        assert s2.run()[r2].output_tokens == done[rid].output_tokens
    assert cache.free_pages() == 6 and cache.free_slots() == 4


def test_request_larger_than_the_pool_fails_cleanly():
    s, model, cache = make(pages=2, ps=4)
    big = s.submit([1] * 9, greedy(1))
    ok = s.submit([1] * 3, greedy(1))
    done = s.run()
    assert done[big].finish_reason == FinishReason.ERROR and "pages" in done[big].error
    assert done[ok].finish_reason == FinishReason.LENGTH
    # a request that fits at first but outgrows the pool alone ends with an error, not a hang
    s, model, cache = make(pages=2, ps=4)
    rid = s.submit([1] * 6, greedy(10))
    done = s.run()
    assert done[rid].finish_reason == FinishReason.ERROR and len(done[rid].output_tokens) >= 1
    assert cache.free_pages() == 2


def test_prefill_portion_shrinks_to_free_pages():
    s, model, cache = make(pages=5, ps=4, budget=64, reqs=4)
    a = s.submit([1] * 12, greedy(3))        # 3 pages, then decodes into a 4th
    s.step()
    b = s.submit([2] * 7, greedy(1))         # admitted with what is free (the pool's last pages)
    o = s.step()
    sizes = {e.rid: len(e.tokens) for e in o.entries}
    assert sizes[a] == 1
    s.run()
    assert s.finished[a].finish_reason == s.finished[b].finish_reason == FinishReason.LENGTH
    cache.check()


def test_temperature_draws_are_reproducible():
    from gibbs_amd.sampling import request_key, uniform
    u = [uniform(5, request_key("r"), i) for i in range(1000)]
    assert all(0.0 <= x < 1.0 for x in u) and abs(sum(u) / 1000 - 0.5) < 0.05
    assert u == [uniform(5, request_key("r"), i) for i in range(1000)]
    assert u[:10] != [uniform(6, request_key("r"), i) for i in range(10)]
    assert u[:10] != [uniform(5, request_key("q"), i) for i in range(10)]


def test_many_requests_that_end_at_admission():
    """More events in one step than the wrapper's buffer was made for (requests that may generate
    nothing end as they reach the head of the queue)."""
    s, model, cache = make(reqs=2)
    rids = [s.submit([1, 2, 3], greedy(0)) for _ in range(200)]
    last = s.submit([4, 5], greedy(1))
    out = s.step()
    assert out.finished[:200] == rids and all(s.finished[r].finish_reason == FinishReason.LENGTH for r in rids)
    assert s.finished[last].output_tokens and not s.has_work()
    assert cache.free_slots() == 2
    cache.check()


def test_preempted_request_does_not_take_the_freed_page_back():
    """Two running requests wait at a page's edge for a page; the youngest, preempted to make room,
    must not take the freed page back at its next admission (it would fill it, be preempted again,
    and the two would wait for ever)."""
    lens, news = [2, 1, 50, 26, 40, 3, 1], [0, 6, 2, 2, 1, 2, 0]
    s, model, cache = make(pages=4, reqs=3, ps=16, budget=3, chunk=16)
    rids = [s.submit([7 + i] * n, greedy(m)) for i, (n, m) in enumerate(zip(lens, news))]
    steps = 0
    while s.has_work():
        s.step()
        cache.check()
        steps += 1
        assert steps < 400, "the scheduler does not get on"
    assert [len(s.finished[r].output_tokens) for r in rids] == news
    assert cache.free_pages() == 4 and cache.free_slots() == 3


def test_random_workloads_always_finish_with_the_tokens_of_a_run_alone():
    """Random pools, budgets and requests, the pool never smaller than the largest request needs:
    every request ends with the tokens it gets alone, nothing is lost, and the number of steps
    stays within what one token per step would take many times over."""
    import random
    for case in range(300):
        rng = random.Random(case)
        ps = rng.choice([2, 4, 16])
        n = rng.randint(1, 8)
        lens = [rng.choice([1, 2, rng.randint(3, 60)]) for _ in range(n)]
        news = [rng.choice([0, 1, rng.randint(2, 30)]) for _ in range(n)]
        most = max(-(-(a + b) // ps) for a, b in zip(lens, news))
        pages = rng.randint(most, most + rng.choice([0, 1, 3, 20]))
        reqs = rng.randint(1, 5)
        budget = rng.choice([1, 2, 3, 8, 64])
        chunk = rng.choice([None, 1, 5, 16])
        if case % 2:
            s, model, cache = make(pages=pages, reqs=reqs, ps=ps, budget=budget, chunk=chunk)
        else:                                    # a second cache group that keeps a window of its keys
            cache = CacheManager([CacheNeed(1, 16), CacheNeed(2, 16, window=rng.choice([1, 3, 8, 20, 50])), None],
                                 [(), (), (StateNeed("s", (2,)),)], ps, pages, reqs)
            model = FakeModel(cache)
            s = ContinuousBatchScheduler(cache, model, context_len=4096, max_batch_tokens=budget, chunk=chunk)
        prompts = [[rng.randint(0, 99) for _ in range(a)] for a in lens]
        rids = [s.submit(p, greedy(m)) for p, m in zip(prompts, news)]
        steps, bound = 0, 50 * (sum(lens) + sum(news)) + 100
        while s.has_work():
            s.step()
            steps += 1
            assert steps < bound, f"case {case}: no end after {steps} steps"
        cache.check()
        assert all(cache.free_pages(g) == pages for g in range(cache.n_groups)) and cache.free_slots() == reqs, f"case {case}"
        for rid, p, m in zip(rids, prompts, news):
            got = s.finished[rid]
            assert got.error is None and len(got.output_tokens) == m, f"case {case}: request {rid}: {got.error}"
            s2, _, _ = make(pages=64, ps=16)
            r2 = s2.submit(p, greedy(m))
            assert s2.run()[r2].output_tokens == got.output_tokens, f"case {case}: request {rid}"


def test_prefill_tuner_budgets():
    """The reference's numbers (src/scheduler/mod.rs:341-403): 64 before anything is
    timed; one token while requests decode and no decode round has been timed; then the tokens that
    cost one decode round, or 100 ms when nothing decodes; at most 2,048; averages move by a quarter."""
    from gibbs_amd.engine.scheduler import PrefillTuner
    t = PrefillTuner()
    assert t.budget(False) == 64 and t.budget(True) == 64
    t.record(0.064, 64, 0)                                   # 1 ms a prompt token
    assert t.budget(False) == 100 and t.budget(True) == 1
    t.record(0.005, 0, 8)                                    # a decode round of 5 ms
    assert t.budget(True) == 5
    t.record(0.009, 0, 8)                                    # 0.75 * 5 + 0.25 * 9 = 6 ms
    assert abs(t.decode_round_s - 0.006) < 1e-12 and t.budget(True) == 6
    t.record(0.012, 6, 8)                                    # beside a decode round: 6 ms for 6 tokens
    assert abs(t.prefill_s_per_token - 0.001) < 1e-12
    fast = PrefillTuner()
    fast.record(1e-6, 1000, 0)
    assert fast.budget(False) == 2048                        # the cap
    slow = PrefillTuner()
    slow.record(1.0, 1, 0); slow.record(0.01, 0, 1)
    assert slow.budget(True) == 1 and slow.budget(False) == 1   # at least one token


def test_measured_budget_through_the_scheduler():
    """`max_batch_tokens="auto"` with a clock that the fake model moves: a prompt token costs 1 ms, a
    step with decoded tokens 4 ms more.  The first step takes 64 prompt tokens; with nothing decoding
    the next ones take 100 (100 ms); beside decoding requests a step takes the 4 tokens that cost
    one decode round."""
    now = [0.0]
    cache = CacheManager([CacheNeed(1, 16), None], [(), (StateNeed("s", (2,)),)], 16, 256, 8)
    model = FakeModel(cache)
    def runner(entries, draws):
        decoded = sum(1 for e in entries if len(e.tokens) == 1 and e.want)
        now[0] += 0.001 * sum(len(e.tokens) for e in entries if not (len(e.tokens) == 1 and e.want)) + (0.004 if decoded else 0)
        return model(entries, draws)
    s = ContinuousBatchScheduler(cache, runner, context_len=4096, max_batch_tokens="auto", clock=lambda: now[0])
    a = s.submit([1] * 300, greedy(40))
    sizes = []
    while len(sizes) < 4:
        o = s.step()
        sizes.append(sum(len(e.tokens) for e in o.entries))
    assert sizes == [64, 100, 100, 36], sizes               # 64 untimed, then 100 ms worth, then the rest
    s.step()                                                 # a decodes: the first decode round is timed
    b = s.submit([2] * 50, greedy(2))
    o = s.step()
    took = {e.rid: len(e.tokens) for e in o.entries}
    assert took[a] == 1 and took[b] == 4, took               # 4 ms a decode round / 1 ms a token
    s.run()
    assert len(s.finished[a].output_tokens) == 40 and len(s.finished[b].output_tokens) == 2
    with pytest.raises(ValueError):
        ContinuousBatchScheduler(cache, runner, context_len=4096, max_batch_tokens="many")
