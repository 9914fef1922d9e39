"""`gibbs --bench SUITE.json`: the reference's suite protocol on this engine.

A suite is `{"defaults": {...}, "models": [{...}, ...]}` (bench/loop.json).  Every
model entry inherits the defaults; the keys that mean something here:

    id              a model folder (config.json + model.safetensors), or "random:CONFIG.json" for
                    random weights of that configuration (seed 0); relative to the suite file
    name            label of the row (default: the folder's or file's name)
    prefill_tokens  length of the timed prompt (default 512)
    decode_tokens   decoded tokens per timed run (default 128)
    runs            timed runs, of which the median counts (default 3)
    batch           requests decoded side by side (default 1)
    dtype           "bfloat16" (default) or "float32"
    min_tok_s       the run fails (exit status 3) if decode is slower
    workload        "decode" (default: the protocol below) or "serve": `requests` prompts of
                    `prefill_tokens` seeded ids each are submitted at once to the continuous-batching
                    scheduler and generate `decode_tokens` tokens each (greedy, no EOS), with
                    `max_requests` live at a time (default: all), prompts cut into portions of at
                    most `chunk` tokens (default: none) under `max_batch_tokens` (default 2048) per
                    step; the row reports generated and prompt tokens a second over the whole run;
                    or "mixed": `batch` requests with `prefill_tokens` cached tokens each decode one token
                    per step beside a prompt portion of `portion` tokens of one more request, through
                    `Engine.step` (no captured graph: what a scheduler step costs); the row reports the
                    wall time of a step and the time after which the host is through with queueing it;
                    or "streams": a kernel that only reads `reads_mib` MiB, and the few-row product of every
                    distinct matrix of the model's layers beside the pure read of its bytes, per kernel of a
                    captured chain
                    or "products": every distinct matrix of the model's layers against `rows`
                    (default 2048) rows of activations, the library's product and the hand-written
                    tiled kernel side by side (`only`: "library" or "own" keeps one of them, for a
                    trace under rocprofv3), each reading its matrix cold as a model step does

Protocol (src/bench.rs:241-322): prompts are seeded synthetic ids (the reference
cycles an encoded sentence to length, :255-259; without tokenizers on this path the ids are drawn
instead); one warm-up prefill, then the median of `runs`; 16 warm-up decode steps, then `runs`
runs of `decode_tokens` steps with sampling on the device, median tokens a second.
`roofline_tok_s = batch * ceiling / bytes a step must read` (:298).  One JSON row per model, then
`METRIC <slug>_tok_s=...` lines and `METRIC geomean_roofline_pct=...` (:522, :739-746).  Exit
status 2 on an error, 3 on a missed `min_tok_s` (:751-757).
"""
from __future__ import annotations

import json
import math
import os
import re
import sys
import time
from typing import Dict, List

DEFAULTS = {"prefill_tokens": 512, "decode_tokens": 128, "runs": 3, "batch": 1, "dtype": "bfloat16"}
WARMUP_STEPS = 16


def _median(xs: List[float]) -> float:
    xs = sorted(xs)
    return xs[len(xs) // 2]


def _slug(name: str) -> str:
    return re.sub(r"[^a-z0-9]+", "_", name.lower()).strip("_")


def _load(entry: Dict, base: str, batch: int = 0, ctx: int = 0):
    import torch

    from .config import config_from_dict
    from .engine import Engine
    from .parts import DecoderModel
    from .weights import random_weights_on_device
    ident = entry["id"]
    if not batch:
        batch = int(entry["batch"])
        ctx = int(entry["prefill_tokens"]) + int(entry["decode_tokens"]) * (int(entry["runs"]) + 1) + WARMUP_STEPS + 64
    if ident.startswith("random:"):
        path = os.path.join(base, ident[len("random:"):])
        with open(path) as f:
            cfg = config_from_dict(json.load(f))
        decls = DecoderModel(cfg.model_spec()).tensor_decls()
        compute = torch.bfloat16 if entry["dtype"] == "bfloat16" else torch.float32
        weights = random_weights_on_device(decls, seed=0, compute_dtype=compute, device="cuda:0")
        return Engine(config=cfg, weights=weights, dtype=entry["dtype"], max_tokens=batch * ctx, max_requests=batch, ctx=ctx)
    path = ident if os.path.isabs(ident) else os.path.join(base, ident)
    return Engine(path, dtype=entry["dtype"], max_tokens=batch * ctx, max_requests=batch, ctx=ctx)


def measure(entry: Dict, base: str) -> Dict:
    import numpy as np
    import torch

    from . import roofline
    from .engine.decode import DecodeLoop
    engine = _load(entry, base)
    vocab = engine.spec.vocab
    n_prompt, n_decode, runs, batch = (int(entry[k]) for k in ("prefill_tokens", "decode_tokens", "runs", "batch"))
    rng = np.random.default_rng(0)

    def prompt():
        return rng.integers(0, vocab, size=n_prompt).tolist()

    times = []
    for _ in range(runs + 1):                                   # the first is the warm-up
        ids = prompt()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        engine.step([("prefill", ids, [n_prompt - 1])])
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
        engine.release("prefill")
    prefill_s = _median(times[1:])

    rids = [f"r{i}" for i in range(batch)]
    first = [int(engine.step([(rid, prompt(), [n_prompt - 1])]).argmax(-1).item()) for rid in rids]
    loop = DecodeLoop(engine, rids, first)
    loop.run(WARMUP_STEPS)
    torch.cuda.synchronize()
    wall, gpu, seq_lens = [], [], []
    for _ in range(runs):
        seq_lens.append([engine.cached_tokens(r) + n_decode // 2 for r in rids])
        loop.prepare(n_decode)              # pages, tables and captured graphs: not in the timed span
        torch.cuda.synchronize()
        begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        begin.record()
        loop.run(n_decode)
        end.record()
        torch.cuda.synchronize()
        wall.append(time.perf_counter() - t0)
        gpu.append(begin.elapsed_time(end) * 1e-3)
    mid = wall.index(_median(wall))
    decode_s = wall[mid]
    step_bytes = roofline.decode_bytes(engine, seq_lens[mid])
    for rid in rids:
        engine.release(rid)
    tok_s = batch * n_decode / decode_s
    roof = batch * roofline.HBM_BYTES_PER_S / step_bytes
    measured = roofline.measured_hbm_bytes_per_s()
    return {"model": entry["name"], "batch": batch, "dtype": entry["dtype"],
            "bytes_per_token": int(step_bytes // batch), "ceiling_gbps": roofline.HBM_BYTES_PER_S / 1e9,
            "decode_tok_s": round(tok_s, 1), "roofline_tok_s": round(roof, 1),
            "roofline_pct": round(100.0 * tok_s / roof, 2),
            # the same against what a kernel that only reads reaches on this GPU (src/bench.rs:438-442)
            "measured_ceiling_gbps": round(measured / 1e9, 1),
            "measured_roofline_pct": round(100.0 * tok_s * step_bytes / batch / measured, 2),
            "wall_ms": round(1e3 * decode_s, 3),
            "ms_per_step": round(1e3 * decode_s / n_decode, 4),
            # per decode step, as the reference's rows have them (src/bench.rs:92-106): the time between the
            # first and the last of the run's launches on the device, what is left of the wall time, and
            # the time the step's bytes take at the ceiling
            "gpu_ms": round(1e3 * gpu[mid] / n_decode, 4), "host_ms": round(1e3 * (decode_s - gpu[mid]) / n_decode, 4),
            "weights_ms": round(1e3 * step_bytes / roofline.HBM_BYTES_PER_S, 4), "prefill_tokens": n_prompt,
            "prefill_tok_s": round(n_prompt / prefill_s, 1),
            "prefill_peak_frac": round(roofline.prefill_flops(engine, n_prompt) / prefill_s
                                       / roofline.PEAK_FLOPS[entry["dtype"]], 4)}


def serve(entry: Dict, base: str) -> Dict:
    """Many requests through the scheduler: what a step holds is the scheduler's decision (prompt
    portions beside decoded tokens, bursts of captured decode steps when only decoding is left)."""
    import numpy as np
    import torch

    from .engine import Generator
    from .sampling import SamplingParams
    n_req, n_prompt, n_decode = int(entry.get("requests", 8)), int(entry["prefill_tokens"]), int(entry["decode_tokens"])
    live = int(entry.get("max_requests", n_req))
    engine = _load(entry, base, batch=live, ctx=-(-(n_prompt + n_decode + 1) // 64) * 64)
    rng = np.random.default_rng(0)
    chunk = entry.get("chunk")
    budget = entry.get("max_batch_tokens", 2048)
    gen = Generator(engine, max_batch_tokens=budget if budget == "auto" else int(budget), chunk=int(chunk) if chunk else None)
    params = SamplingParams(temperature=0.0, max_new_tokens=n_decode, ignore_eos=True)
    # warm-up: as many prompts as fill one step's budget (the library chooses its algorithm for a new
    # number of rows at the first such step), a few decoded tokens each
    per_step = budget if isinstance(budget, int) else 2048
    if chunk:
        per_step = min(per_step, int(chunk))
    n_warm = max(1, min(live, -(-int(per_step) // n_prompt)))
    for _ in range(n_warm):
        gen.submit(rng.integers(0, engine.spec.vocab, size=n_prompt).tolist(),
                   SamplingParams(temperature=0.0, max_new_tokens=20, ignore_eos=True))
    gen.run()
    gen.stats = type(gen.stats)()
    rids = [gen.submit(rng.integers(0, engine.spec.vocab, size=n_prompt).tolist(), params) for _ in range(n_req)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    results = gen.run()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    done = [results[r] for r in rids if r in results and not results[r].error]
    generated = sum(len(r.tokens) for r in done)
    st = gen.stats
    ttft = sorted(r.ttft_s for r in done if r.ttft_s is not None) or [0.0]
    itl = [r.itl_s for r in done if r.itl_s is not None] or [0.0]
    latency = {"ttft_ms_p50": round(1e3 * ttft[len(ttft) // 2], 2), "ttft_ms_max": round(1e3 * ttft[-1], 2),
               "itl_ms_mean": round(1e3 * sum(itl) / len(itl), 3)}
    return {**_serve_row(entry, n_req, live, n_prompt, n_decode, chunk, done, wall, generated, st), **latency}


def products(entry: Dict, base: str) -> Dict:
    """The matrix products of a prompt step one by one: microseconds and PFLOP/s of the library's
    product and of the hand-written tiled kernel for every distinct [out, in] among the model's
    matrices.  Six copies of a matrix take turns, so that every product reads its weights cold."""
    import torch

    from . import ops
    from .config import config_from_dict
    from .parts import DecoderModel
    ident = entry["id"]
    if not ident.startswith("random:"):
        raise ValueError("the products workload takes a configuration (random:CONFIG.json): only shapes matter")
    with open(os.path.join(base, ident[len("random:"):])) as f:
        cfg = config_from_dict(json.load(f))
    model = DecoderModel(cfg.model_spec())
    rows, iters, only = int(entry.get("rows", 2048)), int(entry.get("iters", 24)), entry.get("only")
    shapes: List[tuple] = []
    for block in model.blocks:
        for part in block.parts():
            for shape in part.product_shapes():
                if shape not in shapes:
                    shapes.append(shape)

    def timed(fn) -> float:
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(iters):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / iters * 1e6

    cells = []
    for o, i in shapes:
        x = torch.randn(rows, i, device="cuda:0", dtype=torch.bfloat16)
        ws = [torch.randn(o, i, device="cuda:0", dtype=torch.bfloat16) for _ in range(6)]
        turn = [0]

        def weight():
            turn[0] = (turn[0] + 1) % len(ws)
            return ws[turn[0]]
        flops = 2.0 * rows * o * i
        cell = {"out": o, "in": i}
        if only != "own":
            us = timed(lambda: ops.gemm_library(x, weight()))
            cell.update(library_us=round(us, 1), library_pflops=round(flops / us / 1e9, 3))
        if only != "library":
            us = timed(lambda: ops.gemm_bf16(x, weight(), torch.bfloat16))
            cell.update(own_us=round(us, 1), own_pflops=round(flops / us / 1e9, 3))
        cells.append(cell)
    return {"model": entry["name"], "workload": "products", "dtype": "bfloat16", "rows": rows, "products": cells}


def streams(entry: Dict, base: str) -> Dict:
    """What a kernel that streams a given number of bytes takes inside a chain of dependent kernels (a captured
    graph of 48 launches, the buffers taking turns through 1.5 GiB so that nothing stays cached): a kernel that
    only reads (`reads_mib`), and the few-row products of the decode step for every distinct matrix of the
    model (`rows` rows of X) with the pure read of the same bytes beside them."""
    import torch

    from . import ops
    from .config import config_from_dict
    from .parts import DecoderModel
    dev, chain = "cuda:0", 48
    pool = torch.empty(3 << 28, dtype=torch.bfloat16, device=dev).normal_()          # 1.5 GiB
    pool_bytes = pool.numel() * 2
    sums = torch.zeros(8192, device=dev)

    def per_kernel(fn) -> float:
        fn()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            fn()
        for _ in range(3):
            graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(20):
            graph.replay()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / 20 / chain * 1e6

    def read_us(nbytes: int) -> float:
        nbytes = max(16, nbytes // 16 * 16)
        step = (nbytes + (1 << 20)) // 256 * 256

        def run():
            for i in range(chain):
                ops.probe_read(pool, (i * step) % (pool_bytes - nbytes) // 256 * 256, nbytes, sums)
        return per_kernel(run)

    row = {"model": entry["name"], "workload": "streams", "dtype": "bfloat16",
           "reads": [{"mib": m, "us": round(read_us(int(m * (1 << 20))), 2)} for m in entry.get("reads_mib", [])]}
    ident = entry.get("id")
    if ident:
        if not ident.startswith("random:"):
            raise ValueError("the streams workload takes a configuration (random:CONFIG.json): only shapes matter")
        with open(os.path.join(base, ident[len("random:"):])) as f:
            cfg = config_from_dict(json.load(f))
        model = DecoderModel(cfg.model_spec())
        shapes: List[tuple] = []
        for block in model.blocks:
            for part in block.parts():
                for shape in part.product_shapes():
                    if shape not in shapes:
                        shapes.append(shape)
        n = int(entry.get("rows", 8))
        cells = []
        for o, i in shapes:
            copies = max(2, min(chain, -(-(1 << 29) // (o * i * 2))))       # half a GiB of copies take turns
            ws = [ops.PackedWeight(pool[c * o * i:(c + 1) * o * i].view(o, i)) for c in range(copies)]
            x = torch.randn(n, i, device=dev).to(torch.bfloat16)
            y = torch.empty(n, o, dtype=torch.bfloat16, device=dev)
            us = per_kernel(lambda: [ops.skinny_store(x, ws[c % copies], None, out=y) for c in range(chain)])
            cells.append({"out": o, "in": i, "mib": round(o * i * 2 / (1 << 20), 1), "product_us": round(us, 2),
                          "read_us": round(read_us(o * i * 2), 2)})
            del ws
        row.update(rows=n, products=cells)
    return row


def mixed(entry: Dict, base: str) -> Dict:
    """Steps that hold decoded tokens beside a prompt portion, one after the other without waiting for
    their logits: wall time per step, and how long the host needs to queue one."""
    import numpy as np
    import torch
    n_dec, portion, cached, steps = (int(entry.get(k, d)) for k, d in (("batch", 64), ("portion", 64), ("prefill_tokens", 512),
                                                                         ("steps", 16)))
    ctx = -(-(cached + (steps + 4) * max(portion, 1) + 64) // 64) * 64
    engine = _load(entry, base, batch=n_dec + 1, ctx=ctx)
    rng = np.random.default_rng(0)
    vocab = engine.spec.vocab
    rids = [f"d{i}" for i in range(n_dec)]
    for r in rids:
        engine.step([(r, rng.integers(0, vocab, cached).tolist(), [])])
    engine.step([("p", rng.integers(0, vocab, cached).tolist(), [])])
    feeds = [[(r, [int(t)], [0]) for r, t in zip(rids, rng.integers(0, vocab, n_dec))]
             + ([("p", rng.integers(0, vocab, portion).tolist(), [portion - 1])] if portion else []) for _ in range(steps + 3)]
    for f in feeds[:3]:
        engine.step(f)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for f in feeds[3:]:
        engine.step(f)
    host = time.perf_counter() - t0
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return {"model": entry["name"], "workload": "mixed", "dtype": entry["dtype"], "decoding": n_dec, "portion": portion,
            "rows": n_dec + portion, "cached_tokens": cached,
            "ms_per_step": round(1e3 * wall / steps, 4), "host_ms_per_step": round(1e3 * host / steps, 4)}


def _serve_row(entry, n_req, live, n_prompt, n_decode, chunk, done, wall, generated, st) -> dict:
    return {"model": entry["name"], "workload": "serve", "dtype": entry["dtype"], "requests": n_req, "live": live,
            "prompt_tokens": n_prompt, "decode_tokens": n_decode, "chunk": chunk,
            "finished": len(done), "wall_ms": round(1e3 * wall, 2),
            "decode_tok_s": round(generated / wall, 1), "prompt_tok_s": round(n_req * n_prompt / wall, 1),
            "steps_prefill_ms": round(1e3 * st.prefill_seconds, 2), "steps_decode_ms": round(1e3 * st.decode_seconds, 2),
            "prefill_tok_s": round(st.prefill_tok_s, 1), "decode_only_tok_s": round(st.decode_tok_s, 1)}


def run_suite(path: str) -> int:
    """Runs every model of the suite; returns the process's exit status."""
    try:
        with open(path) as f:
            suite = json.load(f)
        models = suite["models"]
        if not models:
            raise ValueError("the suite names no models")
    except (OSError, ValueError, KeyError) as e:
        print(f"gibbs --bench: cannot read suite {path!r}: {e}", file=sys.stderr)
        return 2
    base = os.path.dirname(os.path.abspath(path))
    rows, missed, failed = [], [], False
    for m in models:
        entry = dict(DEFAULTS)
        entry.update(suite.get("defaults", {}))
        entry.update(m)
        if "id" not in entry and not (entry.get("workload") == "streams" and "name" in entry):
            print("gibbs --bench: a model entry has no id", file=sys.stderr)
            failed = True
            continue
        if "id" in entry:
            ident = entry["id"][len("random:"):] if entry["id"].startswith("random:") else entry["id"]
            entry.setdefault("name", os.path.splitext(os.path.basename(ident.rstrip("/")))[0])
        try:
            workload = entry.get("workload", "decode")
            row = {"serve": serve, "products": products, "mixed": mixed, "streams": streams}.get(workload, measure)(entry, base)
        except Exception as e:     # one model's failure is reported; the others still run (bench.rs:751)
            print(f"gibbs --bench: {entry['name']}: {type(e).__name__}: {e}", file=sys.stderr)
            failed = True
            continue
        rows.append(row)
        print(json.dumps(row), flush=True)
        floor = entry.get("min_tok_s")
        if floor is not None and row.get("decode_tok_s", float("inf")) < float(floor):
            missed.append(f"{row['model']}: {row['decode_tok_s']} tok/s is below min_tok_s {floor}")
    for row in rows:
        if "decode_tok_s" in row:
            print(f"METRIC {_slug(row['model'])}_tok_s={row['decode_tok_s']}")
            print(f"METRIC {_slug(row['model'])}_prefill_tok_s={row['prefill_tok_s']}")
    pcts = [r["roofline_pct"] for r in rows if "roofline_pct" in r]
    if pcts:
        geo = math.exp(sum(math.log(max(p, 1e-9)) for p in pcts) / len(pcts))
        print(f"METRIC geomean_roofline_pct={geo:.2f}")
    for line in missed:
        print(f"gibbs --bench: {line}", file=sys.stderr)
    return 2 if failed else (3 if missed else 0)
