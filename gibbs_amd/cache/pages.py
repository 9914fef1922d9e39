"""Page accounting on the host: a pool of page ids with a free list.

The pool follows the reference's block accounting (/root/reference/src/kv/mod.rs:337-430:
a free list that allocation pops and release pushes), without its reference counts and
prefix tree: a page here belongs to at most one request.  Unlike the reference, whose block
ids are bookkeeping only (/root/reference/src/scheduler/mod.rs:215), these ids index real
device pages that the attention kernels read through a block table.

The pool itself is native code (csrc/host/cache_core.cpp); this class is its handle.
"""
from __future__ import annotations

from typing import Iterable, List, Optional

from . import host


class PageError(RuntimeError):
    """A page was freed twice, freed without being held, or is not of this pool."""


class PagePool:
    def __init__(self, num_pages: int):
        if num_pages <= 0:
            raise ValueError(f"a page pool needs at least one page, not {num_pages}")
        self.num_pages = num_pages
        self._lib = host.library()
        self._pool = self._lib.gibbs_pool_create(num_pages)

    def __del__(self):
        if getattr(self, "_pool", None):
            self._lib.gibbs_pool_destroy(self._pool)
            self._pool = None

    @property
    def n_free(self) -> int:
        return self._lib.gibbs_pool_free(self._pool)

    @property
    def n_held(self) -> int:
        return self.num_pages - self.n_free

    def allocate(self, n: int) -> Optional[List[int]]:
        """`n` pages, or None (and nothing taken) if fewer are free."""
        if n < 0:
            raise ValueError("cannot allocate a negative number of pages")
        out = host.ints([0] * n)
        got = self._lib.gibbs_pool_allocate(self._pool, n, out)
        return None if got < 0 else list(out[:n])

    def release(self, pages: Iterable[int]) -> None:
        pages = list(pages)
        if self._lib.gibbs_pool_release(self._pool, host.ints(pages), len(pages)) < 0:
            raise PageError(host.last_error())

    def is_held(self, page: int) -> bool:
        return bool(self._lib.gibbs_pool_is_held(self._pool, page))
