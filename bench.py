"""Headline benchmark: decode tokens per second of an LFM2-1.2B-shaped model with random weights
on one MI355X (batch 8, 2,048-token prompts, context 4096), with prefill speed at 2,048 tokens and
decode at batch 1 and 64 beside it.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--dtype bfloat16|float32] [--layers L]

A "step" is one decode step of the whole batch.  W untimed steps, then exactly K timed steps
between device synchronisations.  One JSON line is printed.  Protocol after the reference's bench
(/root/reference/src/bench.rs:241-322): warm-up, then timed decode with sampling on the device;
prefill of seeded synthetic ids; roofline = bytes a step must read / bandwidth.
"""
from __future__ import annotations

import argparse
import json
import os
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


def shape_for(layers: int) -> dict:
    cfg = dict(SHAPE)
    if layers != FULL_LAYERS:
        cfg["num_hidden_layers"] = layers
        cfg["full_attn_idxs"] = [i for i in SHAPE["full_attn_idxs"] if i < layers]
    return cfg


def build_engine(dtype: str, layers: int, max_requests: int):
    import torch

    from gibbs_amd import Engine
    from gibbs_amd.config import config_from_dict
    from gibbs_amd.parts import DecoderModel
    from gibbs_amd.weights import random_weights_on_device
    cfg = config_from_dict(shape_for(layers))
    decls = DecoderModel(cfg.model_spec()).tensor_decls()
    compute = torch.bfloat16 if dtype == "bfloat16" else torch.float32
    weights = random_weights_on_device(decls, seed=0, compute_dtype=compute, device="cuda:0")
    return Engine(config=cfg, weights=weights, dtype=dtype, max_tokens=max_requests * CONTEXT,
                  max_requests=max_requests, ctx=CONTEXT)


def seeded_prompt(seed: int, n: int, vocab: int):
    import numpy as np
    return np.random.default_rng(seed).integers(0, vocab, size=n).tolist()


def time_prefill(engine, runs: int = 3):
    """Median time of a whole 2,048-token prompt in one step (one warm-up first)."""
    import torch
    vocab = engine.spec.vocab
    times = []
    for i in range(runs + 1):
        ids = seeded_prompt(1000 + i, PROMPT_LEN, vocab)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        engine.step([("prefill", ids, [PROMPT_LEN - 1])])
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
        engine.release("prefill")
    return sorted(times[1:])[len(times[1:]) // 2]


def time_decode(engine, batch: int, steps: int, warmup: int):
    """Seconds for exactly `steps` decode steps of `batch` requests that each hold a 2,048-token
    prompt; greedy sampling on the device."""
    import torch

    from gibbs_amd.engine.decode import DecodeLoop
    vocab = engine.spec.vocab
    rids = [f"d{i}" for i in range(batch)]
    first = []
    for i, rid in enumerate(rids):
        logits = engine.step([(rid, seeded_prompt(i, PROMPT_LEN, vocab), [PROMPT_LEN - 1])])
        first.append(int(logits.argmax(-1).item()))
    loop = DecodeLoop(engine, rids, first)
    loop.run(warmup)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    loop.run(steps)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    seq_lens = [engine.cached_tokens(r) for r in rids]
    for rid in rids:
        engine.release(rid)
    return dt, seq_lens


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--layers", type=int, default=FULL_LAYERS, help="fewer layers than the shape has (named in config)")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 and 64 points")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU only (this engine has no multi-GPU path); got --gpus {args.gpus}")
        return 2
    if PROMPT_LEN + args.warmup + args.steps + 1 > CONTEXT:
        print(f"--warmup + --steps must stay below {CONTEXT - PROMPT_LEN - 1} (context {CONTEXT})")
        return 2

    from gibbs_amd import roofline as R
    engine = build_engine(args.dtype, args.layers, max_requests=max(64, args.batch))

    prefill_s = time_prefill(engine)
    prefill_flops = R.prefill_flops(engine, PROMPT_LEN)
    peak = R.PEAK_FLOPS[args.dtype]

    dt, seq_lens = time_decode(engine, args.batch, args.steps, args.warmup)
    ms_per_step = dt / args.steps * 1e3
    value = args.batch * args.steps / dt
    # bytes of a decode step at the middle of the timed span
    mid = [n - args.steps // 2 for n in seq_lens]
    step_bytes = R.decode_bytes(engine, mid)
    achieved = step_bytes / (dt / args.steps) / 1e9

    points = {}
    if not args.no_points:
        for b in (1, 64):
            d, _ = time_decode(engine, b, args.steps, args.warmup)
            points[f"decode_b{b}"] = round(b * args.steps / d, 1)

    cfg = engine.config
    line = {
        "metric": f"decode tok/s at batch {args.batch} (LFM2-1.2B shape, 2,048-token prompts, context 4096)",
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic",
        "config": {
            "model": "LFM2-1.2B shape, random weights", "global_batch": args.batch, "seq_len": CONTEXT,
            "parallelism": "single GPU", "prompt_len": PROMPT_LEN, "layers": args.layers,
            "layers_of_shape": FULL_LAYERS, "attention_layers": len(cfg.full_attn_idxs),
            "hidden_size": cfg.hidden_size, "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim, "ff_dim": cfg.intermediate_size, "vocab_size": cfg.vocab_size,
            "conv_L_cache": cfg.conv_L_cache, "tied_head": cfg.tie_embedding, "page_size": engine.page_size,
            "sampling": "greedy on device",
        },
        "prefill": {"value": round(PROMPT_LEN / prefill_s, 1), "tokens": PROMPT_LEN, "ms": round(prefill_s * 1e3, 3),
                    "frac": round(prefill_flops / prefill_s / peak, 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": R.HBM_BYTES_PER_S / 1e9, "unit": "GB/s",
                     "frac": round(achieved / (R.HBM_BYTES_PER_S / 1e9), 4)},
        "points": points,
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
