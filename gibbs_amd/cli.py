"""Command line in the manner of the reference's `gibbs` binary (src/main.rs:27-189):
the same option names and meanings where it has them (`--model`, `--prompt`, `--max-tokens`, `--ctx`,
`--backend`, `--seed`, `--arch`, `--arch-dump`, `--bench`, `--bench-parity`, `--probe-top5`), and this
engine's own beside them (`--replay`, `--random-weights`, sampling and cache options).  One-shot generation prints the reference's lines (main.rs:741-772,
scheduler/mod.rs:1113-1120)."""
from __future__ import annotations

import argparse
import json
import os
import sys
import tempfile
from typing import List, Optional


def parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(prog="gibbs", description="LFM2 inference on one MI355X")
    ap.add_argument("-m", "--model", help="model folder (config.json, model.safetensors[, tokenizer.json])")
    ap.add_argument("--prompt", help="text prompt (needs tokenizer.json in the model folder)")
    ap.add_argument("--prompt-ids", help="prompt as comma-separated token ids")
    ap.add_argument("--max-tokens", type=int, default=None, help="most new tokens (default 64)")
    ap.add_argument("--ctx", type=int, default=None, help="context limit (default: max_position_embeddings, at most 4096)")
    ap.add_argument("--backend", default="auto", help="auto | rocm | hip (cpu is refused: there is no CPU path)")
    ap.add_argument("--seed", type=int, default=0, help="sampling seed (and the seed of --random-weights)")
    ap.add_argument("--arch", help="load --model as this architecture, skipping detection")
    ap.add_argument("--arch-dump", action="store_true",
                    help="print the resolved configuration and the tensor table (JSON), then exit")
    ap.add_argument("--bench", help="benchmark suite (JSON): prints one JSON row per model and METRIC lines")
    ap.add_argument("--bench-parity", action="store_true",
                    help="8 greedy steps in bfloat16 and in float32: same tokens, cosine of the logits >= 0.999")
    ap.add_argument("--replay", metavar="TRACE",
                    help="replay a trace (JSON lines as for bin/trace_run; '-' is standard input) and write logits to --out")
    ap.add_argument("--out", help="folder for the logits of --replay")
    ap.add_argument("--probe-top5", help="print the top-5 next-token logits (JSON) for these comma-separated ids (or a text prompt)")
    ap.add_argument("--temperature", type=float, default=None, help="sampling temperature (one-shot default 0.7; <= 1e-4 is greedy)")
    ap.add_argument("--top-p", type=float, default=None, help="nucleus cut (default 0.9)")
    ap.add_argument("--top-k", type=int, default=50, help="candidates (default 50, at most 64)")
    ap.add_argument("--repetition-penalty", type=float, default=1.0,
                    help="penalty on the tokens among the last 64 (default 1.0: none, as the reference's scheduler passes)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "bf16", "float32", "fp32"])
    ap.add_argument("--random-weights", metavar="CONFIG_JSON",
                    help="write a model folder with random weights from this config.json into --model, then go on")
    ap.add_argument("--max-batch-tokens", type=lambda v: v if v == "auto" else int(v), default=2048,
                    help="prompt tokens per scheduler step, or 'auto': sized by measured costs as the reference's scheduler does")
    ap.add_argument("--chunk", type=int, default=None, help="most prompt tokens of one request per step")
    ap.add_argument("--page-size", type=int, default=None, help="tokens per cache page")
    ap.add_argument("--cache-tokens", type=int, default=None, help="tokens the cache pool holds")
    ap.add_argument("--num-pages", type=int, default=None, help="pages the cache pool holds (instead of --cache-tokens)")
    ap.add_argument("--max-requests", type=int, default=8, help="requests that may be live at once")
    ap.add_argument("--ignore-eos", action="store_true", help="do not stop at an end-of-sequence token")
    return ap


def _tokenizer(model_dir: str):
    from .text import open_text
    return open_text(model_dir)


def _parity(make_engine, prompt: List[int], steps: int = 8) -> int:
    """The reference's device-parity gate (src/bench.rs:761-883: 8 greedy steps on
    Metal and on the CPU, same argmax, cosine >= 0.999), here between the bfloat16 path and the
    true 32-bit path.  The float32 run's tokens are forced on the bfloat16 run so that every step
    compares logits of the same sequence."""
    import torch
    rows = {}
    forced: List[int] = []
    for dt in ("float32", "bfloat16"):
        engine = make_engine(dt)
        logits = [engine.step([("p", prompt, [len(prompt) - 1])])[0].float()]
        for i in range(steps - 1):
            tok = forced[i] if dt == "bfloat16" else int(logits[-1].argmax())
            if dt == "float32":
                forced.append(tok)
            logits.append(engine.step([("p", [tok], [0])])[0].float())
        rows[dt] = torch.stack(logits).cpu()
        del engine
    a, b = rows["float32"], rows["bfloat16"]
    cos = torch.nn.functional.cosine_similarity(a, b, dim=-1)
    same = (a.argmax(-1) == b.argmax(-1))
    ok = bool(same.all()) and float(cos.min()) >= 0.999
    print(json.dumps({"steps": steps, "same_argmax": same.tolist(), "cosine": [round(float(c), 6) for c in cos],
                      "pass": ok}))
    return 0 if ok else 1


def _ids(text: str) -> List[int]:
    return [int(t) for t in text.replace(" ", "").split(",") if t]


def main(argv: Optional[List[str]] = None) -> int:
    args = parser().parse_args(argv)
    if args.backend not in ("auto", "rocm", "hip"):
        print(f"gibbs: backend {args.backend!r} is not available: this engine runs on the GPU only", file=sys.stderr)
        return 2
    if args.bench:
        from .bench_suite import run_suite
        return run_suite(args.bench)
    if not args.model:
        print("gibbs: --model is required", file=sys.stderr)
        return 2

    from .config import config_from_dict, read_config_json
    from .parts import DecoderModel
    from .weights import table_of, write_random_model
    if args.random_weights:
        with open(args.random_weights) as f:
            cfg = config_from_dict(json.load(f), arch=args.arch)
        write_random_model(args.model, cfg, DecoderModel(cfg.model_spec()).tensor_decls(), seed=args.seed)
        print(f"wrote random weights (seed {args.seed}) to {args.model}")
    if args.arch_dump:
        table = table_of(args.model)
        cfg = config_from_dict(read_config_json(args.model), tensors=table, arch=args.arch)
        decls = {d.name for d in DecoderModel(cfg.model_spec()).tensor_decls()}
        print(json.dumps({"architecture": cfg.architecture, "config": cfg.to_dict(),
                          "derived": {"intermediate_size": cfg.intermediate_size, "full_attn_idxs": list(cfg.full_attn_idxs)},
                          "tensors": {n: list(s) for n, s in sorted(table.items())},
                          "unconsumed": sorted(set(table) - decls), "missing": sorted(decls - set(table))}, indent=1))
        return 0

    from .engine import Engine, Generator
    from .sampling import SamplingParams
    from .engine.engine import DEFAULT_PAGE_SIZE
    max_tokens = 64 if args.max_tokens is None else args.max_tokens
    page = args.page_size or DEFAULT_PAGE_SIZE
    pool = args.num_pages * page if args.num_pages else (args.cache_tokens or 16384)
    dtype = {"bf16": "bfloat16", "fp32": "float32"}.get(args.dtype, args.dtype)

    def make_engine(dt):
        return Engine(args.model, dtype=dt, arch=args.arch, ctx=args.ctx, max_requests=args.max_requests,
                      max_tokens=pool, page_size=page)

    if args.bench_parity:
        return _parity(make_engine, _ids(args.prompt_ids) if args.prompt_ids else [1, 2, 3, 4, 5, 6])
    engine = make_engine(dtype)
    if args.replay:
        if not args.out:
            print("gibbs: --replay needs --out", file=sys.stderr)
            return 2
        from .replay import replay
        lines = sys.stdin if args.replay == "-" else open(args.replay)
        replay(engine, lines, args.out)
        return 0
    if args.probe_top5:
        try:
            ids = _ids(args.probe_top5)
        except ValueError:                       # a text prompt, as the reference's probe takes (bench.rs:888-911)
            tok = _tokenizer(args.model)
            if tok is None:
                print("gibbs: --probe-top5 takes token ids, or text when the model folder has tokenizer.json", file=sys.stderr)
                return 2
            ids = tok.prompt_ids(args.probe_top5)
        logits = engine.step([("probe", ids, [len(ids) - 1])])[0]
        top = logits.topk(5)
        print(json.dumps([{"id": int(i), "logit": float(v)} for v, i in zip(top.values.tolist(), top.indices.tolist())]))
        return 0

    tok = _tokenizer(args.model)
    if args.prompt_ids:
        prompt = _ids(args.prompt_ids)
    elif args.prompt is not None:
        if tok is None:
            print("gibbs: --prompt needs tokenizer.json in the model folder; use --prompt-ids", file=sys.stderr)
            return 2
        prompt = tok.prompt_ids(args.prompt)      # through the folder's chat template when it declares one
    else:
        print("gibbs: give --prompt or --prompt-ids", file=sys.stderr)
        return 2
    print(f"💬 Generating from prompt: {args.prompt if args.prompt is not None else prompt!r}")
    declared_greedy = tok is not None and tok.sampling_defaults is not None and tok.sampling_defaults[0] <= 1e-4
    temperature = (0.0 if declared_greedy else 0.7) if args.temperature is None else args.temperature   # main.rs:744-749
    gen = Generator(engine, max_batch_tokens=args.max_batch_tokens, chunk=args.chunk,
                    eos_token_ids=tuple(set(engine.spec.eos_token_ids) | set(tok.stop_ids)) if tok is not None else None)
    rid = gen.submit(prompt, SamplingParams(temperature, args.top_p, args.top_k, max_tokens, args.seed,
                                            args.ignore_eos or tok is None, args.repetition_penalty))
    result = gen.run()[rid]
    st = gen.stats
    print(f"⚡ Prefill: {st.prefill_tokens} tokens in {st.prefill_seconds * 1e3:.2f}ms ({st.prefill_tok_s:.1f} tok/s)")
    text = tok.decode(result.tokens) if tok is not None else " ".join(str(t) for t in result.tokens)
    print(f"✨ Output:\n{text}")
    print(f"⚡ Decode: {st.decode_tokens} tokens in {st.decode_seconds * 1e3:.2f}ms ({st.decode_tok_s:.1f} tok/s) on MI355X (HIP)")
    from .roofline import decode_bytes, HBM_BYTES_PER_S
    nbytes = decode_bytes(engine, [len(prompt) + len(result.tokens)])
    roof = HBM_BYTES_PER_S / nbytes
    if st.decode_tokens:
        print(f"📈 Roofline: {100 * st.decode_tok_s / roof:.1f}% of {roof:.1f} tok/s ({nbytes} B/token at {HBM_BYTES_PER_S / 1e9:.1f} GB/s)")
    if result.error:
        print(f"gibbs: request failed: {result.error}", file=sys.stderr)
        return 1
    return 0


if __name__ == "__main__":
    sys.exit(main())
