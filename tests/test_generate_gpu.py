"""Generation through the entry points: greedy and seeded temperature sampling against the plain
implementation, the reference's golden vector through the engine, continuous batching under
page pressure, the captured decode loop, the replay program and the command line."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from tests import helpers as H
from tests.plain import golden_fixture as G
from tests.plain import lfm2_plain as P

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def dirs(tmp_path_factory):
    root = tmp_path_factory.mktemp("gen")
    out = {n: H.make_model_dir(str(root), n, seed=21 + i) for i, n in enumerate("ABC")}
    G.write_golden_model(str(root / "golden"))
    out["golden"] = str(root / "golden")
    return out


def plain_greedy(model_dir, prompt, n):
    w, cfg = P.load_model_dir(model_dir)
    seq, out = list(prompt), []
    for _ in range(n):
        t = P.argmax_first(P.forward(w, cfg, seq)[-1])
        out.append(t); seq.append(t)
    return out


def acceptable(model_dir, prompt, tokens, dtype) -> int:
    """Every generated token against the plain implementation's choice given the same history.  Where
    the plain logits' best leads the runner-up by more than the engine's logits can be off in this
    precision (two logits, each off by at most the model's measured error: `H.max_logit_error`), the
    token is the plain choice; where the lead is smaller, it is one of the logits that close to the
    best.  Returns the number of tokens that were held to the plain choice."""
    logits = H.plain_logits(model_dir, list(prompt) + list(tokens))
    err = H.max_logit_error(dtype, H.model_of(model_dir)) * np.abs(logits).max()
    exact = 0
    for i, t in enumerate(tokens):
        row = logits[len(prompt) - 1 + i]
        best, runner_up = np.sort(row)[[-1, -2]]
        if best - runner_up > 2 * err:
            exact += 1
            assert t == P.argmax_first(row), f"token {i} = {t}: the plain choice {P.argmax_first(row)} leads by {best - runner_up:.4f} > {2 * err:.4f}"
        else:
            assert row[t] >= best - 2 * err, f"token {i} = {t}: logit {row[t]:.4f} vs best {best:.4f}"
    return exact


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_matches_plain(dirs, dtype):
    from gibbs_amd import Engine, generate
    exact = 0
    for name, lens in (("A", [7, 13]), ("C", [5])):
        eng = Engine(dirs[name], dtype=dtype, max_tokens=512, max_requests=4)
        prompts = [H.tokens(40 + i, n, H.TINY[name]["vocab_size"]) for i, n in enumerate(lens)]
        outs = generate(eng, prompts, max_tokens=16, temperature=0.0, ignore_eos=True)
        for p, o in zip(prompts, outs):
            assert o.finish_reason == "length" and len(o.tokens) == 16
            assert o.ttft_s > 0 and o.itl_s > 0
            if dtype == "float32":
                assert o.tokens == plain_greedy(dirs[name], p, 16)
            exact += acceptable(dirs[name], p, o.tokens, dtype)
        eng.cache.check()
        assert eng.cache.free_slots() == 4
    assert exact >= 10, f"only {exact} of 48 tokens had a lead large enough to be held to the plain choice"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_bursts_change_nothing(dirs, dtype):
    """Generation with bursts of captured decode steps gives the tokens that stepping through the
    host gives: greedy and sampled, requests of different lengths that finish at different times
    (inside bursts that run on until the longest request ends), an end-of-sequence token inside a burst."""
    from gibbs_amd import Engine, Generator, SamplingParams
    d = dirs["B"]
    prompts = [H.tokens(70 + i, n, 512) for i, n in enumerate([9, 21, 5])]
    for temperature in (0.0, 0.9):
        runs = []
        for burst in (0, 5, 16):
            eng = Engine(d, dtype=dtype, max_tokens=1024, max_requests=4)
            gen = Generator(eng, decode_burst=burst, eos_token_ids=())
            rids = [gen.submit(p, SamplingParams(temperature=temperature, max_new_tokens=n, seed=4), rid=f"r{i}")
                    for i, (p, n) in enumerate(zip(prompts, [37, 20, 9]))]
            res = gen.run()
            runs.append([res[r].tokens for r in rids])
            assert [len(t) for t in runs[-1]] == [37, 20, 9]
            if burst == 16:
                # a burst is not cut where the next request reaches its limit: the prompts' step, then 16 + 16 + 4
                # decode steps as three bursts (what the shorter requests sample beyond their limits is dropped)
                assert gen.stats.steps == 4
            eng.cache.check()
            assert eng.cache.free_slots() == 4
        assert runs[0] == runs[1] == runs[2], f"temperature {temperature}"
    # a token that the first request produces mid-way becomes the end token: what follows it is dropped
    # (the same three requests again, so that every kernel sees the batch it saw before)
    stop = runs[0][0][11]
    eng = Engine(d, dtype=dtype, max_tokens=1024, max_requests=4)
    gen = Generator(eng, decode_burst=16, eos_token_ids=(stop,))
    rids = [gen.submit(p, SamplingParams(temperature=0.9, max_new_tokens=n, seed=4), rid=f"r{i}")
            for i, (p, n) in enumerate(zip(prompts, [37, 20, 9]))]
    res = gen.run()
    for i, (rid, full) in enumerate(zip(rids, runs[0])):
        want = full[:full.index(stop)] if stop in full else full
        # (in bfloat16 the others go on in a smaller batch once r0 has stopped, which may round otherwise)
        if i == 0 or dtype == "float32":
            assert res[rid].tokens == want
            assert res[rid].finish_reason == ("stop" if stop in full else "length")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_reference_golden_vector_through_the_engine(dirs, dtype):
    """tests/golden/lm_graphlm_lfm2.json of the reference.  32-bit path: the reference's own golden
    tolerance, rel-L2 < 1e-3 and cos > 0.9999 (tests/golden/util.rs:257-260).  bfloat16 path (the
    fixture's float32 weights are rounded to bfloat16 on loading): the reference's gate for a
    reduced-precision device against its CPU, cosine >= 0.999 (src/bench.rs:761-883)."""
    from gibbs_amd import Engine, Entry, generate
    exp = G.golden_expected()
    eng = Engine(dirs["golden"], dtype=dtype, max_tokens=256, max_requests=2)
    # (bfloat16: 1.5 x the measured relative L2 error of this small model, 3.2 %)
    rel, cos = (1e-3, 0.9999) if dtype == "float32" else (4.8e-2, 0.999)
    def last(rid, ids):
        out = eng.step([Entry(rid, ids, [len(ids) - 1])]).cpu().numpy()[0]
        return out
    for name, ids in (("prefill6", G.PROMPT), ("prefill20", G.LONG_PROMPT)):
        got = last(name, ids)
        H._record(f"golden {name}", "golden", dtype, float(G.rel_l2(got, exp["f32"][name])), float(G.cosine(got, exp["f32"][name])), 0.0)
        assert G.rel_l2(got, exp["f32"][name]) < rel and G.cosine(got, exp["f32"][name]) > cos, name
        eng.release(name)
    last("d", G.PROMPT)
    for i, t in enumerate(G.DECODE):                                    # cached decode of forced tokens
        got = last("d", [t])
        H._record(f"golden decode{i}", "golden", dtype, float(G.rel_l2(got, exp["f32"][f"decode{i}"])), float(G.cosine(got, exp["f32"][f"decode{i}"])), 0.0)
        assert G.rel_l2(got, exp["f32"][f"decode{i}"]) < rel and G.cosine(got, exp["f32"][f"decode{i}"]) > cos
    eng.release("d")
    if dtype == "float32":
        out = generate(eng, [G.PROMPT], max_tokens=8, temperature=0.0, ignore_eos=True)[0]
        assert out.tokens == exp["ids"]["greedy8"]


def test_seeded_temperature_sampling(dirs):
    """The Tiny B workload: four requests (5, 11, 17, 29 tokens), prompt portions of 8,
    temperature 0.8 from a fixed seed.  Every token equals what the plain sampler draws from the
    plain logits of the same history with the same draw."""
    from gibbs_amd import Engine, Generator, SamplingParams
    from gibbs_amd.sampling import request_key, uniform
    d = dirs["B"]
    prompts = [H.tokens(60 + i, n, 512) for i, n in enumerate([5, 11, 17, 29])]
    def run(seed):
        eng = Engine(d, dtype="float32", max_tokens=1024, max_requests=4)
        gen = Generator(eng, max_batch_tokens=16, chunk=8)
        rids = [gen.submit(p, SamplingParams(temperature=0.8, max_new_tokens=12, seed=seed, ignore_eos=True)) for p in prompts]
        res = gen.run()
        return rids, [res[r].tokens for r in rids]
    rids, toks = run(7)
    assert run(7)[1] == toks, "a fixed seed reproduces the tokens"
    assert run(8)[1] != toks
    for rid, p, out in zip(rids, prompts, toks):
        logits = H.plain_logits(d, p + out)
        for i, t in enumerate(out):
            cand, probs = P.nucleus(logits[len(p) - 1 + i].astype(np.float32), 0.8, 50, 0.9)
            assert t == P.draw(cand, probs, uniform(7, request_key(rid), i)), f"request {rid} token {i}"


def test_repetition_penalty_in_generation(dirs):
    """Greedy and sampled requests with a repetition penalty beside a request without one: every
    token is what the plain rule picks from the plain logits of the same history, with the last 64
    tokens of prompt and output as the recent ones; the penalty changes the greedy continuation."""
    from gibbs_amd import Engine, Generator, SamplingParams
    from gibbs_amd.sampling import request_key, uniform
    d = dirs["A"]
    prompts = [H.tokens(50 + i, n, 256) for i, n in enumerate([70, 9, 30])]
    params = [SamplingParams(temperature=0.0, max_new_tokens=24, repetition_penalty=1.7, ignore_eos=True),
              SamplingParams(temperature=0.9, max_new_tokens=24, repetition_penalty=1.3, seed=11, ignore_eos=True),
              SamplingParams(temperature=0.0, max_new_tokens=24, ignore_eos=True)]
    eng = Engine(d, dtype="float32", max_tokens=1024, max_requests=4)
    gen = Generator(eng, max_batch_tokens=32, chunk=16)
    rids = [gen.submit(p, q) for p, q in zip(prompts, params)]
    res = gen.run()
    for rid, p, q in zip(rids, prompts, params):
        out = res[rid].tokens
        logits = H.plain_logits(d, p + out)
        for i, t in enumerate(out):
            row = P.repetition_penalty(logits[len(p) - 1 + i], (p + out[:i])[-64:], q.repetition_penalty, q.greedy)
            if q.greedy:
                best = P.argmax_first(row)
                assert t == best or row[t] >= row[best] - 1e-4, f"request {rid} token {i}"
            else:
                cand, probs = P.nucleus(row, 0.9, 50, 0.9)
                assert t == P.draw(cand, probs, uniform(11, request_key(rid), i)), f"request {rid} token {i}"
    plain = plain_greedy(d, prompts[0], 24)
    assert res[rids[0]].tokens != plain, "a penalty of 1.7 was meant to change the greedy continuation"
    assert res[rids[2]].tokens == plain_greedy(d, prompts[2], 24)


def test_measured_budget_changes_no_token(dirs):
    """`max_batch_tokens="auto"` (the budget sized by measured costs) cuts the prompts elsewhere and
    gives the same tokens; bursts of decode steps feed the measurement too."""
    from gibbs_amd import Engine, Generator, SamplingParams
    d = dirs["B"]
    prompts = [H.tokens(90 + i, n, 512) for i, n in enumerate([150, 9, 77])]
    runs = []
    for budget in (2048, "auto"):
        eng = Engine(d, dtype="float32", max_tokens=2048, max_requests=4)
        gen = Generator(eng, max_batch_tokens=budget)
        rids = [gen.submit(p, SamplingParams(temperature=0.0, max_new_tokens=20, ignore_eos=True)) for p in prompts]
        res = gen.run()
        runs.append([res[r].tokens for r in rids])
        if budget == "auto":
            tuner = gen.scheduler.tuner
            assert tuner.prefill_s_per_token > 0 and tuner.decode_round_s > 0
    assert runs[0] == runs[1]
    # a caller that streams sees every token once, in order, as the steps (or bursts) emit them
    eng = Engine(d, dtype="float32", max_tokens=2048, max_requests=4)
    gen = Generator(eng)
    rids = [gen.submit(p, SamplingParams(temperature=0.0, max_new_tokens=20, ignore_eos=True)) for p in prompts]
    seen = {r: [] for r in rids}
    res = gen.run(on_step=lambda out: [seen[r].append(t) for r, t in out.emitted])
    assert [seen[r] for r in rids] == [res[r].tokens for r in rids] == runs[0]


def test_continuous_batching_under_page_pressure(dirs):
    """A pool so small that running requests collide: the youngest is preempted and recomputed, and
    every request still gets exactly the tokens it gets alone."""
    from gibbs_amd import Engine, Generator, SamplingParams
    d = dirs["A"]
    prompts = [H.tokens(80 + i, n, 256) for i, n in enumerate([20, 24, 18, 30])]
    params = SamplingParams(temperature=0.0, max_new_tokens=24, ignore_eos=True)
    alone = []
    for p in prompts:
        eng = Engine(d, dtype="float32", max_tokens=256, max_requests=1, page_size=8)
        g = Generator(eng)
        r = g.submit(p, params)
        alone.append(g.run()[r].tokens)
    eng = Engine(d, dtype="float32", max_tokens=136, max_requests=4, page_size=8)      # 17 pages for ~200 tokens
    gen = Generator(eng, max_batch_tokens=32)
    rids = [gen.submit(p, params) for p in prompts]
    preempted = 0
    while gen.scheduler.has_work():
        preempted += len(gen.step().preempted)
        eng.cache.check()
    res = gen.results()
    assert preempted > 0, "the pool was meant to be too small"
    for r, want in zip(rids, alone):
        assert res[r].finish_reason == "length" and res[r].tokens == want
    assert eng.cache.free_pages() == 17 and eng.cache.free_slots() == 4


@pytest.mark.parametrize("sampled", [False, True])
def test_requests_that_end_one_after_another_share_padded_decode_loops(dirs, sampled):
    """Five requests of different lengths (one of them ended early by an end-of-sequence token in the
    middle of a burst) decode in captured loops made for 8, 4, 2 and 1 rows: the rows that stand for no
    request are padding in the scratch page and slot.  In 32-bit every request gets exactly the tokens it
    gets alone without bursts; only loops of those row counts were made, and the bursts ran in them."""
    from gibbs_amd import Engine, Generator, SamplingParams
    import importlib
    G_ = importlib.import_module("gibbs_amd.engine.generate")
    d = dirs["B"]
    prompts = [H.tokens(170 + i, n, 512) for i, n in enumerate([9, 21, 5, 14, 30])]
    lengths = [70, 41, 23, 55, 12]
    temperature = 0.9 if sampled else 0.0
    def params(n):
        return SamplingParams(temperature=temperature, max_new_tokens=n, seed=11)
    alone = []
    for i, (p, n) in enumerate(zip(prompts, lengths)):
        eng = Engine(d, dtype="float32", max_tokens=512, max_requests=1)
        g = Generator(eng, decode_burst=0, eos_token_ids=())
        rid = g.submit(p, params(n), rid=f"r{i}")
        alone.append(g.run()[rid].tokens)
    stop = alone[1][17]                                         # request 1 ends here, inside a burst
    cut = alone[1].index(stop)
    eng = Engine(d, dtype="float32", max_tokens=2048, max_requests=5)
    gen = Generator(eng, decode_burst=16, eos_token_ids=(stop,))
    rids = [gen.submit(p, params(n), rid=f"r{i}") for i, (p, n) in enumerate(zip(prompts, lengths))]
    bursts = 0
    while gen.scheduler.has_work():
        before = gen.scheduler.steps
        out = gen.step()
        bursts += gen.scheduler.steps - before > 1
        eng.cache.check()
    res = gen.results()
    for i, r in enumerate(rids):
        want = alone[i]
        if stop in want:
            want = want[:want.index(stop)]
        assert res[r].tokens == want, f"request {i}"
    assert res[rids[1]].finish_reason == "stop" and len(res[rids[1]].tokens) == cut
    made = sorted(rows for rows, _ in gen._loops)
    assert made and set(made) <= set(G_.LOOP_ROWS) and 8 in made, made
    assert bursts >= 4
    assert eng.cache.free_slots() == 5 and eng.cache.free_pages() == eng.cache.pools[0].num_pages


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_loop_graph_replays_match_eager(dirs, dtype):
    """The captured decode step, replayed several times with eager work and synchronisations in
    between, gives on every replay what the eager step function gives."""
    from gibbs_amd import Engine, Entry, SamplingParams
    from gibbs_amd.engine.decode import DecodeLoop
    d = dirs["B"]
    prompts = [H.tokens(90 + i, n, 512) for i, n in enumerate([9, 30, 17])]
    def prefill(eng):
        first = []
        for i, p in enumerate(prompts):
            first.append(int(eng.step([Entry(i, p, [len(p) - 1])]).argmax(-1).item()))
        return first
    # eager reference through the step function, token by token
    eng = Engine(d, dtype=dtype, max_tokens=1024, max_requests=4)
    last, want = prefill(eng), [[] for _ in prompts]
    for _ in range(40):
        logits = eng.step([Entry(i, [last[i]], [0]) for i in range(3)])
        last = logits.argmax(-1).tolist()
        for i in range(3):
            want[i].append(last[i])
    for use_graph in (False, True):
        eng = Engine(d, dtype=dtype, max_tokens=1024, max_requests=4)
        loop = DecodeLoop(eng, [0, 1, 2], prefill(eng), use_graph=use_graph)
        for n in (1, 7, 20, 12):                      # page edges are crossed between and inside runs
            loop.run(n)
            torch.cuda.synchronize()
            eng.step([Entry("other", H.tokens(1, 11, 512), [10])])     # eager work between the replays
            eng.release("other")
        assert loop.tokens() == want, f"use_graph={use_graph}"
        assert [eng.cached_tokens(i) for i in range(3)] == [len(p) + 40 for p in prompts]
    # sampled decoding in the loop equals sampled decoding through the scheduler's sampler
    params = [SamplingParams(temperature=0.9, top_p=0.8, top_k=20, seed=3, ignore_eos=True)] * 3
    eng = Engine(d, dtype=dtype, max_tokens=1024, max_requests=4)
    loop = DecodeLoop(eng, [0, 1, 2], prefill(eng), params=params, first_index=[1, 1, 1])
    loop.run(10); loop.run(6)
    from gibbs_amd.sampling import Draw, Sampler
    eng2 = Engine(d, dtype=dtype, max_tokens=1024, max_requests=4)
    last, sampler, got = prefill(eng2), Sampler(eng2.device), [[] for _ in prompts]
    for s in range(16):
        logits = eng2.step([Entry(i, [last[i]], [0]) for i in range(3)])
        last = sampler.sample(logits, [Draw(params[i], i, 1 + s) for i in range(3)])
        for i in range(3):
            got[i].append(last[i])
    assert loop.tokens() == got


def test_dropped_loops_are_collected_before_a_capture(dirs):
    """A decode loop that was dropped while something still points at it in a cycle is garbage that
    only Python's collector frees; the collector must not get to its graphs while another loop
    captures (a capturing stream refuses the destruction of a graph)."""
    import gc
    from gibbs_amd import Engine, Entry
    from gibbs_amd.engine.decode import DecodeLoop
    d = dirs["A"]
    prompt = H.tokens(3, 12, 256)
    def loop_of(eng, rid):
        first = int(eng.step([Entry(rid, prompt, [len(prompt) - 1])]).argmax(-1).item())
        loop = DecodeLoop(eng, [rid], [first])
        loop.run(9)
        return loop
    eng = Engine(d, dtype="bfloat16", max_tokens=512, max_requests=4)
    old = loop_of(eng, "old")
    want = old.tokens()
    old.cycle = old                       # garbage that reference counting alone does not free
    del old
    threshold = gc.get_threshold()
    gc.set_threshold(1, 1, 1)             # the collector now runs at almost every allocation
    try:
        new = loop_of(eng, "new")
    finally:
        gc.set_threshold(*threshold)
    assert new.tokens() == want and gc.isenabled()


def test_decode_loop_of_more_requests_than_the_fused_path_takes(tmp_path_factory):
    """72 requests decode together: more rows than the fused decode kernels take, so the captured step
    holds the general path with the library's matrix products.  Replays (of one step and of eight),
    with eager work and synchronisations between them, give what eager steps give."""
    from gibbs_amd import Engine, Entry
    from gibbs_amd.engine.decode import DecodeLoop
    d = H.make_model_dir(str(tmp_path_factory.mktemp("medium")), "M", seed=5, std=0.05)
    n = 72
    prompts = [H.tokens(300 + i, 6 + i % 5, 4096) for i in range(n)]
    def prefill(eng):
        return [int(eng.step([Entry(i, p, [len(p) - 1])]).argmax(-1).item()) for i, p in enumerate(prompts)]
    eng = Engine(d, dtype="bfloat16", max_tokens=(n + 1) * 64, max_requests=n + 1)
    last, want = prefill(eng), [[] for _ in prompts]
    for _ in range(20):
        last = eng.step([Entry(i, [last[i]], [0]) for i in range(n)]).argmax(-1).tolist()
        for i in range(n):
            want[i].append(last[i])
    eng = Engine(d, dtype="bfloat16", max_tokens=(n + 1) * 64, max_requests=n + 1)
    loop = DecodeLoop(eng, list(range(n)), prefill(eng))
    for k in (1, 3, 9, 7):
        loop.run(k)
        torch.cuda.synchronize()
        eng.step([Entry("other", H.tokens(1, 11, 4096), [10])])
        eng.release("other")
    assert loop.tokens() == want


def trace_lines(steps):
    return "".join(json.dumps({"step": i, "entries": [{"id": r, "tokens": t, "want": w} for r, t, w in e], "end": end}) + "\n"
                   for i, (e, end) in enumerate(steps))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(dirs, dtype, tmp_path):
    """bin/trace_run as a user runs it: a subprocess fed JSON lines, logits read back from files."""
    d = dirs["A"]
    a, b = H.tokens(1, 70, 256), H.tokens(2, 40, 256)
    steps = [([("a", a[:50], list(range(50)))], []),
             ([("a", a[50:52], [1]), ("b", b[:33], [0, 32])], []),
             ([("b", b[33:35], [])], []),                                   # nothing wanted: no file
             ([("a", a[52:53], [0]), ("b", b[35:40], [4])], ["b"]),
             ([("a", a[53:70], list(range(17)))], ["a"])]
    out = tmp_path / "logits"
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", d, "--dtype", dtype,
                           "--out", str(out), "--max-tokens", "192"], input=trace_lines(steps), capture_output=True,
                          text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(5)]
    assert not (out / "2.f32").exists()
    pa, pb = H.plain_logits(d, a), H.plain_logits(d, b)
    read = lambda i: np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, 256)
    H.assert_close(read(0), pa[:50], dtype, "step 0")
    H.assert_close(read(1), np.stack([pa[51], pb[0], pb[32]]), dtype, "step 1")
    H.assert_close(read(3), np.stack([pa[52], pb[39]]), dtype, "step 3")
    H.assert_close(read(4), pa[53:70], dtype, "step 4")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program_four_ways(dirs, dtype, tmp_path):
    """The program itself (a subprocess, JSON lines in, files out) over the four ways of running the same
    requests of Tiny B: whole; most in one step and the last 32 tokens one by one; portions of changing
    size down to two tokens; mixed, up to four live requests in a pool so small that pages are used
    again (--max-tokens 4 x 128).  Every wanted place against the plain implementation."""
    from tests.test_engine_gpu import mixed_schedule, portions
    d = dirs["B"]
    vocab = H.TINY["B"]["vocab_size"]
    seqs = {f"q{i}": H.tokens(900 + i, n, vocab) for i, n in enumerate([100, 45, 90, 64, 81, 50, 77, 96])}
    assert sum(-(-len(s) // 16) for s in seqs.values()) > 512 // 16, "the pool must be too small to avoid reuse"
    first = seqs["q0"]
    ways = {
        "whole": [([(r, ids, list(range(len(ids))))], [r]) for r, ids in seqs.items()],
        "tail": [([("q0", first[:68], list(range(68)))], [])] + [([("q0", [t], [0])], []) for t in first[68:]] + [([], ["q0"])],
        "portions": [([("q0", first[a:b], list(range(b - a)))], []) for a, b in portions(100, [7, 2, 13, 3, 2, 33, 5, 2, 17])],
        "mixed": mixed_schedule(seqs, np.random.default_rng(12)),
    }
    for way, steps in ways.items():
        out = tmp_path / way
        proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", d, "--dtype", dtype,
                               "--out", str(out), "--max-tokens", "512"], input=trace_lines(steps), capture_output=True,
                              text=True, timeout=300)
        assert proc.returncode == 0, proc.stderr[-2000:]
        assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(len(steps))]
        at, got, want = {}, [], []
        for i, (entries, ends) in enumerate(steps):
            wanted = sum(len(w) for _, _, w in entries)
            if wanted:
                got.append(np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(wanted, vocab))
                want += [H.plain_logits(d, seqs[r])[at.get(r, 0) + w] for r, _, places in entries for w in places]
            for r, toks, _ in entries:
                at[r] = at.get(r, 0) + len(toks)
            for r in ends:
                at.pop(r, None)
        places = len(want)
        H.assert_close(np.concatenate(got), np.stack(want), dtype, f"trace_run {way}", model="B")
        assert places >= 100, way


def test_command_line(dirs, tmp_path):
    env = dict(os.environ)
    run = lambda *a: subprocess.run([sys.executable, os.path.join(ROOT, "bin", "gibbs"), *a], capture_output=True,
                                    text=True, timeout=300, env=env)
    prompt = H.tokens(5, 9, 256)
    p = run("--model", dirs["A"], "--prompt-ids", ",".join(map(str, prompt)), "--max-tokens", "6", "--temperature", "0",
            "--dtype", "float32")
    assert p.returncode == 0, p.stderr[-2000:]
    assert "⚡ Prefill: 9 tokens" in p.stdout and "⚡ Decode: 5 tokens" in p.stdout and "📈 Roofline:" in p.stdout
    line = p.stdout.split("✨ Output:\n")[1].splitlines()[0]
    assert [int(t) for t in line.split()] == plain_greedy(dirs["A"], prompt, 6)
    p = run("--model", dirs["B"], "--arch-dump")
    dump = json.loads(p.stdout)
    assert dump["architecture"] == "Lfm2ForCausalLM" and dump["unconsumed"] == [] and dump["missing"] == []
    assert dump["derived"] == {"intermediate_size": 256, "full_attn_idxs": [0, 2, 5]}
    p = run("--model", dirs["A"], "--probe-top5", "1,2,3", "--dtype", "float32")
    top = json.loads(p.stdout.strip().splitlines()[-1])
    want = H.plain_logits(dirs["A"], [1, 2, 3])[-1]
    assert [t["id"] for t in top] == np.argsort(-want)[:5].tolist()
    assert run("--model", dirs["A"], "--prompt-ids", "1", "--backend", "cpu").returncode == 2
    # a text prompt: through the folder's tokenizer and chat template, decoded on the way out
    import pathlib
    import shutil
    from tests.test_text import TEMPLATE, write_folder
    texted = pathlib.Path(shutil.copytree(dirs["A"], tmp_path / "texted"))
    write_folder(texted, template=TEMPLATE, generation={"do_sample": False}, write_config=False)
    p = run("--model", str(texted), "--prompt", "hello world", "--max-tokens", "5", "--ignore-eos", "--dtype", "float32")
    assert p.returncode == 0, p.stderr[-2000:]
    assert "⚡ Prefill: 5 tokens" in p.stdout, "BOS, the user marker, two words and the assistant marker"
    want = plain_greedy(dirs["A"], [1, 3, 5, 6, 4], 5)        # the folder declares greedy decoding
    from gibbs_amd.text import open_text
    assert p.stdout.split("✨ Output:\n")[1].splitlines()[0] == open_text(str(texted)).decode(want)
    cfgfile = tmp_path / "cfg.json"
    cfgfile.write_text(json.dumps(H.TINY["C"]))
    p = run("--model", str(tmp_path / "fresh"), "--random-weights", str(cfgfile), "--seed", "5", "--prompt-ids", "3,4",
            "--max-tokens", "3")
    assert p.returncode == 0 and os.path.isfile(tmp_path / "fresh" / "model.safetensors"), p.stderr[-2000:]


def test_command_line_replay_and_parity(dirs, tmp_path):
    run = lambda *a, **k: subprocess.run([sys.executable, os.path.join(ROOT, "bin", "gibbs"), *a], capture_output=True,
                                         text=True, timeout=300, env=dict(os.environ), **k)
    toks = H.tokens(11, 20, 256)
    trace = [{"step": 0, "entries": [{"id": "a", "tokens": toks[:12], "want": [11]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": toks[12:], "want": [0, 7]}], "end": ["a"]}]
    (tmp_path / "trace.jsonl").write_text("".join(json.dumps(t) + "\n" for t in trace))
    p = run("--model", dirs["A"], "--dtype", "fp32", "--replay", str(tmp_path / "trace.jsonl"), "--out",
            str(tmp_path / "logits"), "--num-pages", "8")
    assert p.returncode == 0 and p.stdout.split() == ["done", "0", "done", "1"], p.stderr[-2000:]
    want = H.plain_logits(dirs["A"], toks)
    got = np.fromfile(tmp_path / "logits" / "1.f32", dtype="<f4").reshape(2, -1)
    H.assert_close(got, want[[12, 19]], "float32", "replay through the command line")
    assert run("--model", dirs["A"], "--replay", "-", input="").returncode == 2          # no --out
    p = run("--model", dirs["A"], "--bench-parity", "--prompt-ids", ",".join(map(str, toks[:9])))
    row = json.loads(p.stdout.strip().splitlines()[-1])
    assert row["steps"] == 8 and len(row["cosine"]) == 8 and min(row["cosine"]) >= 0.999
    assert p.returncode == (0 if row["pass"] else 1) and row["pass"] == all(row["same_argmax"])


def test_bench_suite_through_the_command_line(dirs, tmp_path):
    """`gibbs --bench SUITE.json`: one JSON row per model, METRIC lines, and the reference's exit
    statuses (3 for a missed min_tok_s, 2 for a suite that cannot be run)."""
    run = lambda *a: subprocess.run([sys.executable, os.path.join(ROOT, "bin", "gibbs"), *a], capture_output=True,
                                    text=True, timeout=300, env=dict(os.environ))
    (tmp_path / "cfg.json").write_text(json.dumps(H.TINY["C"]))
    suite = {"defaults": {"prefill_tokens": 40, "decode_tokens": 8, "runs": 2},
             "models": [{"id": dirs["A"], "name": "Tiny A", "dtype": "float32"},
                        {"id": "random:cfg.json", "batch": 3},
                        {"id": dirs["B"], "name": "served", "workload": "serve", "requests": 5, "max_requests": 3,
                         "prefill_tokens": 21, "decode_tokens": 12, "chunk": 8, "max_batch_tokens": 16}]}
    (tmp_path / "suite.json").write_text(json.dumps(suite))
    p = run("--bench", str(tmp_path / "suite.json"))
    assert p.returncode == 0, p.stderr[-2000:]
    rows = [json.loads(l) for l in p.stdout.splitlines() if l.startswith("{")]
    assert [r["model"] for r in rows] == ["Tiny A", "cfg", "served"] and rows[1]["batch"] == 3
    served = rows.pop()
    assert served["finished"] == 5 and served["live"] == 3 and served["decode_tok_s"] > 0 and served["prompt_tok_s"] > 0
    assert 0 < served["ttft_ms_p50"] <= served["ttft_ms_max"] and served["itl_ms_mean"] > 0
    for r in rows:
        assert r["decode_tok_s"] > 0 and r["prefill_tok_s"] > 0 and 0 < r["roofline_pct"] < 100
        assert abs(r["roofline_tok_s"] * r["bytes_per_token"] - r["ceiling_gbps"] * 1e9) < 1e-3 * r["ceiling_gbps"] * 1e9
    assert "METRIC tiny_a_tok_s=" in p.stdout and "METRIC cfg_prefill_tok_s=" in p.stdout
    assert "METRIC geomean_roofline_pct=" in p.stdout
    suite["models"][0]["min_tok_s"] = 1e12
    (tmp_path / "suite.json").write_text(json.dumps(suite))
    p = run("--bench", str(tmp_path / "suite.json"))
    assert p.returncode == 3 and "below min_tok_s" in p.stderr
    assert run("--bench", str(tmp_path / "absent.json")).returncode == 2
    suite["models"].append({"id": str(tmp_path / "no_such_model")})
    (tmp_path / "suite.json").write_text(json.dumps(suite))
    assert run("--bench", str(tmp_path / "suite.json")).returncode == 2
