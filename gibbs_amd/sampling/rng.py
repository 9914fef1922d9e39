"""Counter-based random numbers for sampling: the draw of output token `index` of a request is a
pure function of (seed, request key, index), so a fixed seed reproduces the tokens whatever else
runs beside the request and however often it was preempted and recomputed.

The reference derives its draw from a hash of the recent tokens and the candidate set, without a
seed (src/runtime/lm.rs:1126-1137); a seeded stream replaces that here.  The
mixer is SplitMix64, which the reference's device sampler also uses
(src/graph/metal_kernels.metal:2369-2460).
"""
from __future__ import annotations

import hashlib

MASK = (1 << 64) - 1


def splitmix64(x: int) -> int:
    x = (x + 0x9E3779B97F4A7C15) & MASK
    z = x
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & MASK
    return z ^ (z >> 31)


def request_key(rid) -> int:
    """A stable 64-bit key of a request id (an int is its own key)."""
    if isinstance(rid, int):
        return rid & MASK
    return int.from_bytes(hashlib.sha256(repr(rid).encode()).digest()[:8], "little")


def uniform(seed: int, key: int, index: int) -> float:
    """u in [0, 1) with 24 bits, exactly representable in float32."""
    x = splitmix64((seed & MASK) ^ splitmix64(key ^ splitmix64(index & MASK)))
    return (x >> 40) / float(1 << 24)
