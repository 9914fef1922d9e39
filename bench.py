"""Headline benchmark: decode tokens per second of an LFM2-1.2B-shaped model with random weights
on one MI355X (batch 8, 2,048-token prompts, context 4096), with prefill speed at 2,048 tokens and
decode at batch 1 and 64 beside it.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--dtype bfloat16|float32] [--layers L]
                    [--batch B] [--prompt-len P --context C] [--suite bench/SUITE.json]

`--prompt-len` / `--context` move the same measurement to longer contexts (16k, 32k, 100k);
`--prefill-tokens` times a prompt of another length than 2,048; `--page-size` another page size than the engine's 16; `--suite` runs the rows of a suite file of `gibbs --bench` afterwards
(the serving workloads of the 350M and 2.6B shapes in bench/lfm2.json) and puts them into the line
under `rows`.

A "step" is one decode step of the whole batch.  W untimed steps, then runs of exactly K timed steps
between device synchronisations: the median of 3 runs counts (src/bench.rs:274-296).  Before a timed
run its pages are reserved and both captured graphs exist, so the span holds replays only, whatever W
is.  One JSON line is printed.  Protocol after the reference's bench (src/bench.rs:241-322): warm-up,
then timed decode with sampling on the device; prefill of seeded synthetic ids; roofline = bytes a step
must read / bandwidth.  Beside the speed, as the reference's bench has it (src/bench.rs:761-883), a
correctness gate (`parity`): a 3-layer model of the same layer sizes, 64 prompt tokens and 8 forced
decode steps, the 32-bit path against the plain implementation under tests/ and the bfloat16 path
against the 32-bit path; and the kernels that the decode step's time goes to (`top_kernels`,
src/bench.rs:114-115).
"""
from __future__ import annotations

import argparse
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# the LFM2-1.2B shape (Liquid's 1.2B model: 16 layers, 6 of them attention)
SHAPE = dict(
    architectures=["Lfm2ForCausalLM"], model_type="lfm2", hidden_size=2048, num_hidden_layers=16,
    full_attn_idxs=[2, 5, 8, 10, 12, 14], num_attention_heads=32, num_key_value_heads=8, head_dim=64,
    block_ff_dim=12288, block_auto_adjust_ff_dim=True, block_ffn_dim_multiplier=1.0, block_multiple_of=256,
    vocab_size=65536, tie_embedding=True, conv_L_cache=3, conv_bias=False, rope_theta=1000000.0,
    norm_eps=1e-5, max_position_embeddings=128000)
PROMPT_LEN = 2048
CONTEXT = 4096
FULL_LAYERS = 16
RUNS = 3


def shape_for(layers: int) -> dict:
    cfg = dict(SHAPE)
    if layers != FULL_LAYERS:
        cfg["num_hidden_layers"] = layers
        cfg["full_attn_idxs"] = [i for i in SHAPE["full_attn_idxs"] if i < layers]
    return cfg


def build_engine(dtype: str, layers: int, max_requests: int, context: int = CONTEXT, page_size: int = 0):
    import torch

    from gibbs_amd import Engine
    from gibbs_amd.config import config_from_dict
    from gibbs_amd.parts import DecoderModel
    from gibbs_amd.weights import random_weights_on_device
    cfg = config_from_dict(shape_for(layers))
    decls = DecoderModel(cfg.model_spec()).tensor_decls()
    compute = torch.bfloat16 if dtype == "bfloat16" else torch.float32
    weights = random_weights_on_device(decls, seed=0, compute_dtype=compute, device="cuda:0")
    return Engine(config=cfg, weights=weights, dtype=dtype, max_tokens=max_requests * context,
                  max_requests=max_requests, ctx=context, **({"page_size": page_size} if page_size else {}))


def seeded_prompt(seed: int, n: int, vocab: int):
    import numpy as np
    return np.random.default_rng(seed).integers(0, vocab, size=n).tolist()


def time_prefill(engine, runs: int = 5, n_tokens: int = PROMPT_LEN, warmups: int = 3):
    """Median time of a whole prompt of `n_tokens` (2,048 unless asked otherwise) in one step.  Three untimed steps
    first: the first holds the library's choice of algorithms, and the next two still run 5 to 10 % slower than the
    steady state that follows (clocks, caches)."""
    import torch
    vocab = engine.spec.vocab
    times = []
    for i in range(warmups + runs):
        ids = seeded_prompt(1000 + i, n_tokens, vocab)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        engine.step([("prefill", ids, [n_tokens - 1])])
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
        engine.release("prefill")
    timed = sorted(times[warmups:])
    return timed[len(timed) // 2]


def time_decode(engine, batch: int, steps: int, warmup: int, runs: int = RUNS, profile: bool = False,
                prompt_len: int = PROMPT_LEN):
    """Median seconds for exactly `steps` decode steps of `batch` requests that each hold a
    `prompt_len`-token prompt (greedy sampling on the device), the requests' lengths at the middle of that
    run, and, with `profile`, the kernels of one more run by their share of its device time."""
    import torch

    from gibbs_amd.engine.decode import DecodeLoop
    vocab = engine.spec.vocab
    rids = [f"d{i}" for i in range(batch)]
    first = []
    for i, rid in enumerate(rids):
        logits = engine.step([(rid, seeded_prompt(i, prompt_len, vocab), [prompt_len - 1])])
        first.append(int(logits.argmax(-1).item()))
    loop = DecodeLoop(engine, rids, first)
    if warmup > 0:
        loop.run(warmup)
    samples = []
    for _ in range(runs):
        loop.prepare(steps)                 # pages, tables and both captured graphs: not in the timed span
        lens = [engine.cached_tokens(r) + steps // 2 for r in rids]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        loop.run(steps)
        torch.cuda.synchronize()
        samples.append((time.perf_counter() - t0, lens))
    top = kernel_shares(lambda: loop.run(min(steps, 16))) if profile else None
    for rid in rids:
        engine.release(rid)
    dt, seq_lens = sorted(samples, key=lambda s: s[0])[len(samples) // 2]
    return dt, seq_lens, top


def kernel_shares(run, most: int = 8):
    """Runs `run()` under the profiler and returns the kernels that its device time goes to:
    [{"name", "calls", "us", "share"}], largest first, or None where the profiler gives no device
    times."""
    import torch
    from torch.profiler import ProfilerActivity, profile
    try:
        with profile(activities=[ProfilerActivity.CPU, ProfilerActivity.CUDA]) as prof:
            run()
            torch.cuda.synchronize()
        rows = [(e.key, e.count, float(getattr(e, "device_time_total", 0.0) or getattr(e, "cuda_time_total", 0.0)))
                for e in prof.key_averages()
                if str(getattr(e, "device_type", "")).endswith("CUDA")]
    except Exception as exc:                                   # the figures are an extra: the bench line stands without them
        print(f"bench: no kernel shares ({type(exc).__name__}: {exc})", file=sys.stderr)
        return None
    total = sum(us for _, _, us in rows)
    if total <= 0:
        return None
    merged = {}
    for name, calls, us in rows:
        short = name.replace("(anonymous namespace)::", "").replace("void ", "").split("(")[0].strip()
        mangled = re.match(r"_Z(?:N\d+_GLOBAL__N_1)?(\d+)", short)      # a name the profiler left mangled: keep the identifier
        if mangled:
            start = mangled.end()
            short = short[start:start + int(mangled.group(1))]
        entry = merged.setdefault(short[:72] or name[:72], [0, 0.0])
        entry[0] += int(calls)
        entry[1] += us
    ranked = sorted(merged.items(), key=lambda kv: -kv[1][1])[:most]
    return [{"name": name, "calls": calls, "us": round(us, 1), "share": round(us / total, 4)}
            for name, (calls, us) in ranked]


def suite_rows(path: str) -> list:
    """The rows of a `gibbs --bench` suite file, measured here one after the other (a row that fails
    is reported with its error)."""
    import gc

    import torch

    from gibbs_amd import bench_suite as S
    with open(path) as f:
        suite = json.load(f)
    base = os.path.dirname(os.path.abspath(path))
    rows = []
    for m in suite["models"]:
        entry = dict(S.DEFAULTS, **suite.get("defaults", {}), **m)
        ident = entry["id"][len("random:"):] if entry["id"].startswith("random:") else entry["id"]
        entry.setdefault("name", os.path.splitext(os.path.basename(ident.rstrip("/")))[0])
        try:
            rows.append({"serve": S.serve, "products": S.products, "mixed": S.mixed}.get(entry.get("workload", "decode"), S.measure)(entry, base))
        except Exception as exc:
            rows.append({"model": entry["name"], "error": f"{type(exc).__name__}: {exc}"})
        gc.collect()
        torch.cuda.empty_cache()
    return rows


PARITY_PROMPT, PARITY_DECODE = 64, 8
# bfloat16 against the 32-bit path at these layer sizes: the largest difference of a logit measured is
# 0.9 % of the largest logit (3 layers); a place whose best logit leads by more than twice the bound
# must keep its choice
PARITY_BF16_MAX_ERR = 0.02


def greedy_through_loop(engine, prompt, n: int) -> list:
    """`n` greedy tokens after `prompt` through the captured decode loop (the path that the speed
    figures time: the rows' embeddings written by the end of the step before, argmax on the device)."""
    from gibbs_amd.engine.decode import DecodeLoop
    first = int(engine.step([("g", prompt, [len(prompt) - 1])]).argmax(-1).item())
    loop = DecodeLoop(engine, ["g"], [first])
    loop.run(n - 1)
    out = [first] + loop.tokens()[0]
    engine.release("g")
    return out


def greedy_through_steps(engine, prompt, n: int) -> list:
    out = [int(engine.step([("s", prompt, [len(prompt) - 1])]).argmax(-1).item())]
    for _ in range(n - 1):
        out.append(int(engine.step([("s", [out[-1]], [0])]).argmax(-1).item()))
    engine.release("s")
    return out


def parity(layers: int = 3) -> dict:
    """The correctness gate beside the speed figures (src/bench.rs:761-883: 8 greedy steps, same
    argmax, cosine >= 0.999), at the benchmark's layer sizes with `layers` layers (a convolution,
    an attention and a convolution layer): a model folder with random weights is written, 64 prompt
    tokens run as one step and 8 given tokens one by one; the logits of those 9 places from the
    32-bit path are held against the plain implementation's (at most 1e-5 of the scale, same
    argmax), and the bfloat16 path's against the 32-bit path's (cosine >= 0.999, no logit further off
    than `PARITY_BF16_MAX_ERR` of the scale, the same argmax wherever the 32-bit lead is more than
    twice that).  Then 8 greedy tokens through the captured decode loop, the path that is timed: in
    32-bit they are the plain implementation's, in bfloat16 those of the same engine stepped from
    the host."""
    import tempfile

    import numpy as np

    from gibbs_amd import Engine
    from gibbs_amd.config import config_from_dict
    from gibbs_amd.parts import DecoderModel
    from gibbs_amd.weights import write_random_model
    from tests.plain import lfm2_plain as P
    shape = dict(SHAPE, num_hidden_layers=layers, full_attn_idxs=[1])
    cfg = config_from_dict(shape)
    ids = seeded_prompt(77, PARITY_PROMPT + PARITY_DECODE, cfg.vocab_size)
    prompt = ids[:PARITY_PROMPT]
    with tempfile.TemporaryDirectory() as tmp:
        write_random_model(tmp, cfg, DecoderModel(cfg.model_spec()).tensor_decls(), seed=5, gain_std=0.1)
        got, loop_tokens, step_tokens = {}, {}, {}
        for dtype in ("float32", "bfloat16"):
            engine = Engine(tmp, dtype=dtype, max_tokens=512, max_requests=2, ctx=256)
            rows = [engine.step([("p", prompt, [PARITY_PROMPT - 1])])[0]]
            rows += [engine.step([("p", [t], [0])])[0] for t in ids[PARITY_PROMPT:]]
            got[dtype] = np.stack([r.float().cpu().numpy() for r in rows]).astype(np.float64)
            engine.release("p")
            loop_tokens[dtype] = greedy_through_loop(engine, prompt, PARITY_DECODE)
            step_tokens[dtype] = greedy_through_steps(engine, prompt, PARITY_DECODE)
            del engine
        weights, raw = P.load_model_dir(tmp)
        want = P.forward(weights, raw, ids)[PARITY_PROMPT - 1:]
        seq, plain_tokens = list(prompt), []
        for _ in range(PARITY_DECODE):
            plain_tokens.append(P.argmax_first(P.forward(weights, raw, seq)[-1]))
            seq.append(plain_tokens[-1])
    f32, b16 = got["float32"], got["bfloat16"]
    scale = np.abs(want).max()
    err = float(np.abs(f32 - want).max() / scale)
    cos = (f32 * b16).sum(-1) / np.sqrt((f32 * f32).sum(-1) * (b16 * b16).sum(-1))
    rel = float(np.sqrt(((b16 - f32) ** 2).sum(-1) / (f32 ** 2).sum(-1)).max())
    b16_err = float(np.abs(b16 - f32).max() / scale)
    same_f32 = int((f32.argmax(-1) == want.argmax(-1)).sum())
    top2 = np.sort(f32, axis=-1)[:, -2:]
    decided = (top2[:, 1] - top2[:, 0]) > 2 * PARITY_BF16_MAX_ERR * scale
    same_b16 = int((b16.argmax(-1) == f32.argmax(-1))[decided].sum())
    n = len(want)
    loop_ok = loop_tokens["float32"] == plain_tokens and loop_tokens["bfloat16"] == step_tokens["bfloat16"]
    ok = (err <= 1e-5 and same_f32 == n and float(cos.min()) >= 0.999 and b16_err <= PARITY_BF16_MAX_ERR
          and same_b16 == int(decided.sum()) and loop_ok)
    return {"layers": layers, "places": n, "fp32_vs_plain_max_err_of_scale": float(f"{err:.3e}"),
            "fp32_same_argmax": same_f32, "bf16_vs_fp32_min_cosine": round(float(cos.min()), 6),
            "bf16_vs_fp32_max_rel_l2": round(rel, 5), "bf16_vs_fp32_max_err_of_scale": round(b16_err, 5),
            "bf16_same_argmax": same_b16, "bf16_places_with_a_clear_lead": int(decided.sum()),
            "fp32_loop_tokens_are_plain": loop_tokens["float32"] == plain_tokens,
            "bf16_loop_tokens_are_stepped": loop_tokens["bfloat16"] == step_tokens["bfloat16"], "pass": bool(ok)}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--layers", type=int, default=FULL_LAYERS, help="fewer layers than the shape has (named in config)")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prompt-len", type=int, default=PROMPT_LEN, help="tokens every request holds before decoding starts")
    ap.add_argument("--context", type=int, default=None, help="context limit (default 4096, or what --prompt-len needs)")
    ap.add_argument("--prefill-tokens", type=int, default=PROMPT_LEN, help="length of the timed prompt (default 2,048)")
    ap.add_argument("--page-size", type=int, default=0, help="tokens per cache page (default: the engine's, 16)")
    ap.add_argument("--suite", help="a suite file of `gibbs --bench` whose rows are run afterwards and reported under `rows`")
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 and 64 points")
    ap.add_argument("--no-parity", action="store_true", help="skip the correctness gate")
    ap.add_argument("--no-kernels", action="store_true", help="skip the kernels' shares of the decode step")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU only (this engine has no multi-GPU path); got --gpus {args.gpus}")
        return 2
    if args.steps < 1 or args.warmup < 0:
        print("--steps must be at least 1 and --warmup at least 0")
        return 2
    need = max(args.prompt_len + args.warmup + (RUNS + 1) * args.steps + 1, args.prefill_tokens)
    context = args.context or max(CONTEXT, -(-need // 1024) * 1024)
    if args.prompt_len < 1 or need > context:
        print(f"--prompt-len + --warmup + {RUNS + 1} x --steps must stay below the context ({context})")
        return 2

    from gibbs_amd import roofline as R
    gate = None if args.no_parity else parity()
    engine = build_engine(args.dtype, args.layers, max_requests=args.batch if args.no_points else max(64, args.batch),
                          context=context, page_size=args.page_size)

    ceiling = R.measured_hbm_bytes_per_s()
    prefill_s = time_prefill(engine, n_tokens=args.prefill_tokens)
    prefill_flops = R.prefill_flops(engine, args.prefill_tokens)
    peak = R.PEAK_FLOPS[args.dtype]

    dt, seq_lens, top = time_decode(engine, args.batch, args.steps, args.warmup, profile=not args.no_kernels,
                                    prompt_len=args.prompt_len)
    ms_per_step = dt / args.steps * 1e3
    value = args.batch * args.steps / dt
    # bytes of a decode step at the middle of the timed span
    step_bytes = R.decode_bytes(engine, seq_lens)
    achieved = step_bytes / (dt / args.steps) / 1e9

    points = {}
    if not args.no_points:
        for b in (1, 64):
            d, _, _ = time_decode(engine, b, args.steps, args.warmup, prompt_len=args.prompt_len)
            points[f"decode_b{b}"] = round(b * args.steps / d, 1)

    cfg = engine.config
    line = {
        "metric": f"decode tok/s at batch {args.batch} (LFM2-1.2B shape, {args.prompt_len:,}-token prompts, context {context})",
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic",
        "config": {
            "model": "LFM2-1.2B shape, random weights", "global_batch": args.batch, "seq_len": context,
            "parallelism": "single GPU", "prompt_len": args.prompt_len, "layers": args.layers,
            "layers_of_shape": FULL_LAYERS, "attention_layers": len(cfg.full_attn_idxs),
            "hidden_size": cfg.hidden_size, "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim, "ff_dim": cfg.intermediate_size, "vocab_size": cfg.vocab_size,
            "conv_L_cache": cfg.conv_L_cache, "tied_head": cfg.tie_embedding, "page_size": engine.page_size,
            "sampling": "greedy on device", "timed_runs": RUNS,
        },
        "prefill": {"value": round(args.prefill_tokens / prefill_s, 1), "tokens": args.prefill_tokens, "ms": round(prefill_s * 1e3, 3),
                    "frac": round(prefill_flops / prefill_s / peak, 4)},
        # `peak` is the published figure; `measured_peak` is what a kernel that only reads reaches on this GPU
        # (the reference's rows divide by a measured ceiling, src/bench.rs:438-442)
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": R.HBM_BYTES_PER_S / 1e9, "unit": "GB/s",
                     "frac": round(achieved / (R.HBM_BYTES_PER_S / 1e9), 4), "measured_peak": round(ceiling / 1e9, 1),
                     "frac_of_measured": round(achieved / (ceiling / 1e9), 4)},
        "points": points, "parity": gate, "top_kernels": top,
    }
    if args.suite:
        del engine
        line["rows"] = suite_rows(args.suite)
    if gate is not None and not gate["pass"]:
        # speed of an engine that fails its correctness gate is no measurement: the figures stay in the
        # line for the reader, under another key, and the run fails
        line["value_with_failed_parity"], line["value"] = line["value"], None
        print(json.dumps(line))
        return 3
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
