"""Times the matrix products of a prompt step, the library's against the hand-written tiled kernel:

    python -m gibbs_amd.bench_gemm [--rows 2048] [--shapes 16384x2048,2048x8192,...] [--only library|own]

Weights are rotated through several buffers so that every product reads its matrix cold, as a model
step does.  One line per shape: microseconds and PFLOP/s of each.  Under `rocprofv3` the same run gives
the kernels' counters (`--only` keeps one of the two in the trace).
"""
from __future__ import annotations

import argparse
import time

# out x in of the LFM2-1.2B shape's products: w1|w3, w2, in_proj, out_proj, qkv
DEFAULT_SHAPES = "16384x2048,2048x8192,6144x2048,2048x2048,3072x2048"


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="bench_gemm", description=__doc__.split("\n\n")[0])
    ap.add_argument("--rows", type=int, default=2048, help="rows of the activations (tokens of the step)")
    ap.add_argument("--shapes", default=DEFAULT_SHAPES, help="comma-separated OUTxIN")
    ap.add_argument("--only", choices=["library", "own"], help="time only one of the two")
    ap.add_argument("--iters", type=int, default=24)
    args = ap.parse_args(argv)
    import torch

    from . import ops
    dev = "cuda:0"

    def timed(fn) -> float:
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.iters):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / args.iters * 1e6

    for shape in args.shapes.split(","):
        o, i = (int(v) for v in shape.lower().split("x"))
        x = torch.randn(args.rows, i, device=dev, dtype=torch.bfloat16)
        ws = [torch.randn(o, i, device=dev, dtype=torch.bfloat16) for _ in range(6)]
        turn = [0]

        def weight():
            turn[0] = (turn[0] + 1) % len(ws)
            return ws[turn[0]]
        flops = 2.0 * args.rows * o * i
        cells = []
        if args.only != "own":
            us = timed(lambda: ops.gemm_library(x, weight()))
            cells.append(f"library {us:7.1f} us {flops / us / 1e9:5.2f} PFLOP/s")
        if args.only != "library":
            us = timed(lambda: ops.gemm_bf16(x, weight(), torch.bfloat16))
            cells.append(f"own {us:7.1f} us {flops / us / 1e9:5.2f} PFLOP/s")
        print(f"rows {args.rows:5d}  {o:6d} x {i:5d}: " + " | ".join(cells), flush=True)
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
