"""The cache manager: pages and block tables per request and cache group, and slots for
per-request state of fixed size.

Groups.  Layers whose mixers have the same `CacheNeed` share a group.  A group owns one page
pool; page p of the group is the same slot in every layer's key and value pages, so one block
table per request serves all layers of the group.  A group with a window gives pages back as
soon as every position in them has fallen out of the window of all later queries.

Slots.  Every live request holds one slot; the state of every layer that keeps state of fixed
size lives at that slot index of the layer's state tensor.  A slot is cleared when a request
takes it.

What is given back and when.  `release` returns every page and the slot (a request finished,
failed or was preempted); `commit` returns a window group's passed pages.  Pages are used
again without being cleared: kernels see a key only through its position, never through what
a page holds.  The reference returns blocks on the same events
(src/scheduler/mod.rs:1215-1217, :1561-1563).
"""
from __future__ import annotations

from typing import Dict, Hashable, List, Optional, Sequence, Tuple, Union

import numpy as np

from . import host
from .needs import CacheNeed, StateNeed

NO_PAGE = -1


class PageError(RuntimeError):
    """A page was freed twice, freed without being held, or is not of its pool."""


class _PoolView:
    """What the rest of the package asks of a group's pool."""

    def __init__(self, manager: "CacheManager", group: int, num_pages: int):
        self._manager, self._group, self.num_pages = manager, group, num_pages

    @property
    def n_free(self) -> int:
        return self._manager.free_pages(self._group)

    @property
    def n_held(self) -> int:
        return self.num_pages - self.n_free


class CacheManager:
    """Host-side accounting, kept by the native core (csrc/host/cache_core.cpp); this class maps
    request ids to the core's slots and turns its failure codes into exceptions.  Device tensors
    hang on `DeviceCache`, which reads this."""

    def __init__(self, needs: Sequence[Optional[CacheNeed]], states: Sequence[Sequence[StateNeed]],
                 page_size: int, num_pages: Union[int, Sequence[int]], max_requests: int):
        """`needs[i]` / `states[i]`: what the mixer of run i of the layer order asks for (None / ()
        for nothing).  `num_pages`: pages of every group's pool, or one count per group in the
        order the groups first appear (a group with a window can do with fewer)."""
        if page_size <= 0 or max_requests <= 0:
            raise ValueError("page_size and max_requests must be positive")
        self.page_size = page_size
        self.max_requests = max_requests
        self.group_needs: List[CacheNeed] = []
        self.group_layers: List[List[int]] = []
        self.layer_group: Dict[int, int] = {}
        for i, need in enumerate(needs):
            if need is None:
                continue
            if need not in self.group_needs:
                self.group_needs.append(need)
                self.group_layers.append([])
            g = self.group_needs.index(need)
            self.group_layers[g].append(i)
            self.layer_group[i] = g
        n_groups = len(self.group_needs)
        per_group = [int(num_pages)] * n_groups if isinstance(num_pages, int) else [int(n) for n in num_pages]
        if len(per_group) != n_groups:
            raise ValueError(f"{len(per_group)} page counts for {n_groups} cache groups")
        if any(n <= 0 for n in per_group):
            raise ValueError(f"a page pool needs at least one page, not {min(per_group)}")
        # state layout of a slot: (layer, name) -> (offset in 4-byte words, shape, type)
        self.state_layout: Dict[Tuple[int, str], Tuple[int, Tuple[int, ...], str]] = {}
        off = 0
        for i, layer_states in enumerate(states):
            for s in layer_states:
                if (i, s.name) in self.state_layout:
                    raise ValueError(f"layer {i} declares state {s.name!r} twice")
                self.state_layout[(i, s.name)] = (off, tuple(s.shape), s.dtype)
                off += s.words
        self.slot_floats = off        # 4-byte words of a slot
        self._lib = host.library()
        windows = host.ints([int(n.window or 0) for n in self.group_needs])
        self._core = self._lib.gibbs_cache_create(n_groups, windows, page_size, host.ints(per_group), max_requests)
        if not self._core:
            raise ValueError("the cache core refused its sizes")
        self.pools = [_PoolView(self, g, per_group[g]) for g in range(n_groups)]
        self._slots: Dict[Hashable, int] = {}
        self._needed = host.ints([0] * len(self.group_needs))

    def __del__(self):
        if getattr(self, "_core", None):
            self._lib.gibbs_cache_destroy(self._core)
            self._core = None

    def _raise(self, code: int, rid: Hashable = None):
        text = host.last_error()
        if rid is not None:
            text = f"request {rid!r}: {text}"
        if code == host.ERR_PAGE:
            raise PageError(text)
        raise ValueError(text)

    # ------------------------------------------------------------------ queries
    @property
    def n_groups(self) -> int:
        return len(self.group_needs)

    @property
    def core(self):
        """The native core (for the step staging of the engine)."""
        return self._core

    def __contains__(self, rid: Hashable) -> bool:
        return rid in self._slots

    def live(self) -> List[Hashable]:
        return list(self._slots)

    def tokens(self, rid: Hashable) -> int:
        return self._lib.gibbs_cache_tokens(self._core, self._slots[rid])

    def slot(self, rid: Hashable) -> int:
        return self._slots[rid]

    def free_pages(self, group: int = 0) -> int:
        return self._lib.gibbs_cache_free_pages(self._core, group)

    def free_slots(self) -> int:
        return self._lib.gibbs_cache_free_slots(self._core)

    def pages_for(self, n_tokens: int) -> int:
        return -(-n_tokens // self.page_size)

    def pages_needed(self, rid: Hashable, n_new: int) -> List[int]:
        """Per group: pages that `reserve(rid, n_new)` would have to take."""
        self._lib.gibbs_cache_pages_needed(self._core, self._slots[rid], n_new, self._needed)
        return list(self._needed[:self.n_groups])

    # ------------------------------------------------------------------ life of a request
    def admit(self, rid: Hashable) -> bool:
        """Gives the request a slot (cleared before the next step); False if none is free."""
        if rid in self._slots:
            raise KeyError(f"request {rid!r} is already live")
        slot = self._lib.gibbs_cache_admit(self._core)
        if slot < 0:
            return False
        self._slots[rid] = slot
        return True

    def reserve(self, rid: Hashable, n_new: int) -> bool:
        """Pages for the next `n_new` positions in every group; all or nothing."""
        code = self._lib.gibbs_cache_reserve(self._core, self._slots[rid], n_new)
        if code == host.ERR_NO_ROOM:
            return False
        if code < 0:
            self._raise(code, rid)
        return True

    def reserve_all(self, rids: Sequence[Hashable], n_new: int, limit: int = 0) -> Optional[bool]:
        """Pages for the next `n_new` positions of every one of the requests, all or nothing, in one call of the
        core: True if pages were taken, False if none were needed, None if they do not fit (`pages_needed_all` then
        says how many every group would have needed).  `limit`: the positions a request may hold (0: no check)."""
        slots = host.ints([self._slots[r] for r in rids])
        code = self._lib.gibbs_cache_reserve_all(self._core, slots, len(rids), n_new, limit, self._needed)
        self.pages_needed_all = list(self._needed[:self.n_groups])
        if code == host.ERR_NO_ROOM:
            return None
        if code < 0:
            self._raise(code, rids[0] if rids else None)
        return code > 0

    def commit_all(self, rids: Sequence[Hashable], n_new: int) -> None:
        """`n_new` more positions of every one of the requests are cached now."""
        code = self._lib.gibbs_cache_commit_all(self._core, host.ints([self._slots[r] for r in rids]), len(rids), n_new)
        if code < 0:
            self._raise(code, rids[0] if rids else None)

    def commit(self, rid: Hashable, n_new: int) -> None:
        """`n_new` more positions are cached now.  A window group gives back every page that
        no later query can see: page j holds positions [j*ps, (j+1)*ps), the next query is at
        position >= tokens and sees keys > tokens - window."""
        code = self._lib.gibbs_cache_commit(self._core, self._slots[rid], n_new)
        if code < 0:
            self._raise(code, rid)

    def release(self, rid: Hashable) -> None:
        """Gives back every page and the slot of a request that ended."""
        slot = self._slots.pop(rid)
        code = self._lib.gibbs_cache_release(self._core, slot)
        if code < 0:
            self._raise(code, rid)

    def adopt(self, rid: Hashable, slot: int) -> None:
        """The native scheduler admitted `rid` into `slot` of the core: learn the name."""
        if rid in self._slots:
            raise KeyError(f"request {rid!r} is already live")
        self._slots[rid] = slot

    def forget(self, rid: Hashable) -> None:
        """The native scheduler gave the request's slot and pages back."""
        del self._slots[rid]

    # ------------------------------------------------------------------ what kernels read
    def slots_of(self, rids: Sequence[Hashable]):
        return host.ints([self._slots[r] for r in rids])

    def table_width(self, rids: Sequence[Hashable], group: int) -> int:
        return max(0, self._lib.gibbs_cache_table_width(self._core, self.slots_of(rids), len(rids), group))

    def block_table(self, rids: Sequence[Hashable], group: int, width: Optional[int] = None) -> np.ndarray:
        """int32 [len(rids), width]: page id of logical page j of each request (NO_PAGE beyond
        its pages and for pages a window has passed)."""
        width = max(1, self.table_width(rids, group)) if width is None else width
        out = np.empty((len(rids), width), dtype=np.int32)
        code = self._lib.gibbs_cache_block_table(self._core, self.slots_of(rids), len(rids), group, width,
                                                 out.ctypes.data)
        if code < 0:
            self._raise(code)
        return out

    def take_fresh_slots(self) -> List[int]:
        """Slots that requests have taken since the last call (every one of them, once)."""
        out, fresh = host.ints([0] * self.max_requests), []
        while True:
            n = self._lib.gibbs_cache_take_fresh_slots(self._core, out, self.max_requests)
            fresh += list(out[:n])
            if n < self.max_requests:
                return fresh

    # ------------------------------------------------------------------ invariants (tests)
    def check(self) -> None:
        """No page lost, held twice or free while held; no slot shared or lost."""
        code = self._lib.gibbs_cache_check(self._core)
        if code < 0:
            self._raise(code)
        if len(set(self._slots.values())) != len(self._slots):
            raise PageError("two requests share a slot")
        if len(self._slots) + self.free_slots() != self.max_requests:
            raise PageError("a slot was lost")
