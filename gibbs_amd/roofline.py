"""What a step must at least move and compute, for the roofline figures of the bench and the
command line (the reference reports decode speed against bytes-per-token at a bandwidth ceiling,
src/bench.rs:298-308)."""
from __future__ import annotations

from typing import Sequence

# MI355X's published peaks.
HBM_BYTES_PER_S = 8.0e12
PEAK_FLOPS = {"bfloat16": 2.5e15, "float16": 2.5e15, "float8": 5.0e15, "float32": 157.3e12}


_measured_ceiling = None


def measured_hbm_bytes_per_s(mib: int = 512, pool_mib: int = 2048, repeats: int = 5) -> float:
    """What a kernel that only reads reaches on this GPU: `mib` MiB read by a plain sum kernel, the read
    window moving through a pool of `pool_mib` MiB so that nothing is found in a cache, the best of
    `repeats` timed by device events.  The reference divides by a measured streaming ceiling rather
    than the spec-sheet figure (src/bench.rs:438-442); the rows report both.  Measured once per process."""
    global _measured_ceiling
    if _measured_ceiling is None:
        import torch

        from . import ops
        pool = torch.empty(pool_mib << 19, dtype=torch.bfloat16, device="cuda").normal_()
        sums = torch.zeros(4096, device="cuda")
        nbytes, pool_bytes = mib << 20, pool_mib << 20
        best = 0.0
        for r in range(repeats + 1):                           # the first is the warm-up
            offset = (r * nbytes) % (pool_bytes - nbytes + 1) // 256 * 256
            begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            begin.record()
            ops.probe_read(pool, offset, nbytes, sums, grid=4096, block=256)
            end.record()
            torch.cuda.synchronize()
            if r:
                best = max(best, nbytes / (begin.elapsed_time(end) * 1e-3))
        del pool
        _measured_ceiling = best
    return _measured_ceiling


def torch_element_size(dtype) -> int:
    import torch
    return torch.empty((), dtype=dtype).element_size()


def _nbytes(t) -> int:
    return t.numel() * t.element_size()


def weight_bytes_per_step(engine) -> int:
    """Every weight a decode step uses, once: the matrices and small tensors of every run of the
    layer order, the final norm and the head matrix.  (The token table is read by rows only,
    unless it is also the head.)"""
    m = engine.model
    total = 0
    for i in m.spec.order:
        b = m.blocks[i]
        total += sum(_nbytes(t) for t in b.matrices()) + sum(_nbytes(t) for t in b.small_tensors())
    total += sum(_nbytes(t) for t in m.final_norm.small_tensors())
    total += _nbytes(m.head)
    return total


def cache_bytes(engine, seq_lens: Sequence[int]) -> int:
    """Keys and values that the live requests' next tokens attend over, and their state slots."""
    cm = engine.cache
    elem = torch_element_size(engine.device_cache.cache_dtype)
    total = 0
    for g, need in enumerate(cm.group_needs):
        per_token = need.kv_heads * (need.head_dim + need.value_dim) * elem * len(cm.group_layers[g])
        for n in seq_lens:
            total += per_token * (n if need.window is None else min(n, need.window))
    total += len(seq_lens) * cm.slot_floats * 4
    return total


def decode_bytes(engine, seq_lens: Sequence[int]) -> int:
    return weight_bytes_per_step(engine) + cache_bytes(engine, seq_lens)


def prefill_flops(engine, n_tokens: int, n_logit_rows: int = 1, start: int = 0) -> float:
    """Multiply-adds x 2 of a prompt portion of `n_tokens` rows starting at position `start`:
    every matrix once per row, the head for the wanted rows, and causal attention (each row over
    the keys up to its own position)."""
    m = engine.model
    flops = 0.0
    keys = sum(start + t + 1 for t in range(n_tokens))
    for i in m.spec.order:
        b = m.blocks[i]
        flops += 2.0 * n_tokens * sum(t.numel() for t in b.matrices())
        flops += b.attention_flops(keys)
    flops += 2.0 * n_logit_rows * m.head.numel()
    return flops
