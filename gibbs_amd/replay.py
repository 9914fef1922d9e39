"""Trace replay: feeds given token ids through a model step by step and writes logits.

It samples nothing and owns no model code: every step goes through `Engine.step`, the step
function that generation uses, with the engine's own cache manager and kernels.

Input (standard input, one JSON object a line):
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
For a step in which something is wanted, `<out>/<step>.f32` holds the logits at the wanted
places, in the order of the entries and of `want`, as little-endian float32 [wanted, vocab].
After every step a line `done <step>` is printed and flushed.
"""
from __future__ import annotations

import argparse
import json
import os
import sys


def replay(engine, lines, out_dir: str, report=print) -> None:
    """Runs the steps of `lines` (JSON objects, one a line) through `engine.step`."""
    from .engine import Entry
    os.makedirs(out_dir, exist_ok=True)
    for line in lines:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        step = rec["step"]
        entries = [Entry(e["id"], e["tokens"], e.get("want", [])) for e in rec.get("entries", [])]
        if entries:
            logits = engine.step(entries)
            if logits is not None:
                arr = logits.detach().to("cpu").numpy().astype("<f4", copy=False)
                tmp = os.path.join(out_dir, f".{step}.f32.tmp")
                arr.tofile(tmp)
                os.replace(tmp, os.path.join(out_dir, f"{step}.f32"))
        for rid in rec.get("end", []):
            if rid in engine.cache:
                engine.release(rid)
        report(f"done {step}", flush=True)


def pool_tokens_for(max_tokens: int, page: int) -> int:
    """Every request's count is rounded up to a multiple of max(64, page size)."""
    unit = max(64, page)
    return -(-max_tokens // unit) * unit


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16",
                    help="bfloat16: the kernels and precisions that serving uses; float32: everything in true 32-bit")
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens that live requests hold at any time (each rounded up to whole pages)")
    ap.add_argument("--page-size", type=int, default=None, help="tokens per cache page (default: the engine's)")
    ap.add_argument("--max-requests", type=int, default=8, help="state slots (live requests)")
    args = ap.parse_args(argv)

    print("trace_run: loading kernels and model", file=sys.stderr, flush=True)
    from .engine import Engine
    from .engine.engine import DEFAULT_PAGE_SIZE

    from .config import config_from_dict, read_config_json
    from .weights import table_of
    page = args.page_size or DEFAULT_PAGE_SIZE
    # a trace may be as long as the model allows (generation's default context limit is shorter)
    longest = config_from_dict(read_config_json(args.model), tensors=table_of(args.model)).model_spec().max_position
    engine = Engine(args.model, dtype=args.dtype, max_tokens=pool_tokens_for(args.max_tokens, page),
                    max_requests=args.max_requests, page_size=page, ctx=longest)
    print("trace_run: ready", file=sys.stderr, flush=True)
    replay(engine, sys.stdin, args.out)
    return 0


if __name__ == "__main__":
    sys.exit(main())
