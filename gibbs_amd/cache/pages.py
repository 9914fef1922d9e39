"""Page accounting on the host: a pool of page ids with a free list.

The pool follows the reference's block accounting (/root/reference/src/kv/mod.rs:337-430:
a free list that allocation pops and release pushes), without its reference counts and
prefix tree: a page here belongs to at most one request.  Unlike the reference, whose block
ids are bookkeeping only (/root/reference/src/scheduler/mod.rs:215), these ids index real
device pages that the attention kernels read through a block table.
"""
from __future__ import annotations

from typing import Iterable, List, Optional


class PageError(RuntimeError):
    """A page was freed twice, freed without being held, or is not of this pool."""


class PagePool:
    def __init__(self, num_pages: int):
        if num_pages <= 0:
            raise ValueError(f"a page pool needs at least one page, not {num_pages}")
        self.num_pages = num_pages
        # LIFO: a page that was just given back is the next to be used again.
        self._free: List[int] = list(range(num_pages - 1, -1, -1))
        self._held = [False] * num_pages

    @property
    def n_free(self) -> int:
        return len(self._free)

    @property
    def n_held(self) -> int:
        return self.num_pages - len(self._free)

    def allocate(self, n: int) -> Optional[List[int]]:
        """`n` pages, or None (and nothing taken) if fewer are free."""
        if n < 0:
            raise ValueError("cannot allocate a negative number of pages")
        if n > len(self._free):
            return None
        out = [self._free.pop() for _ in range(n)]
        for p in out:
            self._held[p] = True
        return out

    def release(self, pages: Iterable[int]) -> None:
        for p in pages:
            if not 0 <= p < self.num_pages:
                raise PageError(f"page {p} is not of this pool (0..{self.num_pages - 1})")
            if not self._held[p]:
                raise PageError(f"page {p} freed twice or never held")
            self._held[p] = False
            self._free.append(p)

    def is_held(self, page: int) -> bool:
        return self._held[page]
