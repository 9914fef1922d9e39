"""What a mixer asks of the cache manager: paged keys and values, and fixed-size state."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple


@dataclass(frozen=True)
class CacheNeed:
    """Keys and values of every cached position (`window` None), or of the last `window`
    positions only.  Layers with equal needs form one group: one page pool and one block
    table per request serve all of them.  Values may have a head size of their own
    (`v_head_dim`, default: the keys')."""
    kv_heads: int
    head_dim: int
    window: Optional[int] = None
    v_head_dim: Optional[int] = None

    @property
    def value_dim(self) -> int:
        return self.head_dim if self.v_head_dim is None else self.v_head_dim


STATE_DTYPES = {"float32": 4, "int32": 4, "bfloat16": 2, "float16": 2}


@dataclass(frozen=True)
class StateNeed:
    """A tensor of fixed shape per request (for instance a short convolution's last K-1 inputs), kept in the
    request's slot: float32 unless the mixer names another type of `STATE_DTYPES`.  A slot is a row of 4-byte
    words; every state starts at a word, and a slot is all zero bits when a request takes it."""
    name: str
    shape: Tuple[int, ...]
    dtype: str = "float32"

    def __post_init__(self):
        if self.dtype not in STATE_DTYPES:
            raise ValueError(f"state {self.name!r}: type {self.dtype!r} is none of {sorted(STATE_DTYPES)}")

    @property
    def numel(self) -> int:
        n = 1
        for s in self.shape:
            n *= s
        return n

    @property
    def words(self) -> int:
        """4-byte words of a slot that the state takes."""
        return -(-self.numel * STATE_DTYPES[self.dtype] // 4)
