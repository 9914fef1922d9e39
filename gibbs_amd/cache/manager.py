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
(/root/reference/src/scheduler/mod.rs:1215-1217, :1561-1563).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

import numpy as np

from .needs import CacheNeed, StateNeed
from .pages import PageError, PagePool

NO_PAGE = -1


@dataclass
class _Request:
    slot: int
    tokens: int = 0                                         # positions whose keys/state are cached
    pages: Dict[int, List[int]] = field(default_factory=dict)   # group -> logical page -> id or NO_PAGE


class CacheManager:
    """Host-side accounting.  Device tensors hang on `DeviceCache`, which reads this."""

    def __init__(self, needs: Sequence[Optional[CacheNeed]], states: Sequence[Sequence[StateNeed]],
                 page_size: int, num_pages: int, max_requests: int):
        """`needs[i]` / `states[i]`: what the mixer of run i of the layer order asks for (None / ()
        for nothing).  `num_pages`: pages of every group's pool."""
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
        self.pools = [PagePool(num_pages) for _ in self.group_needs]
        # state layout of a slot: (layer, name) -> (offset, shape), in float32 elements
        self.state_layout: Dict[Tuple[int, str], Tuple[int, Tuple[int, ...]]] = {}
        off = 0
        for i, layer_states in enumerate(states):
            for s in layer_states:
                if (i, s.name) in self.state_layout:
                    raise ValueError(f"layer {i} declares state {s.name!r} twice")
                self.state_layout[(i, s.name)] = (off, tuple(s.shape))
                off += s.numel
        self.slot_floats = off
        self._free_slots = list(range(max_requests - 1, -1, -1))
        self._requests: Dict[Hashable, _Request] = {}
        self.fresh_slots: List[int] = []            # slots taken since the device last cleared them

    # ------------------------------------------------------------------ queries
    @property
    def n_groups(self) -> int:
        return len(self.group_needs)

    def __contains__(self, rid: Hashable) -> bool:
        return rid in self._requests

    def live(self) -> List[Hashable]:
        return list(self._requests)

    def tokens(self, rid: Hashable) -> int:
        return self._requests[rid].tokens

    def slot(self, rid: Hashable) -> int:
        return self._requests[rid].slot

    def free_pages(self, group: int = 0) -> int:
        return self.pools[group].n_free

    def free_slots(self) -> int:
        return len(self._free_slots)

    def pages_for(self, n_tokens: int) -> int:
        return -(-n_tokens // self.page_size)

    def pages_needed(self, rid: Hashable, n_new: int) -> List[int]:
        """Per group: pages that `reserve(rid, n_new)` would have to take."""
        r = self._requests[rid]
        want = self.pages_for(r.tokens + n_new)
        return [max(0, want - len(r.pages[g])) for g in range(self.n_groups)]

    # ------------------------------------------------------------------ life of a request
    def admit(self, rid: Hashable) -> bool:
        """Gives the request a slot (cleared before the next step); False if none is free."""
        if rid in self._requests:
            raise KeyError(f"request {rid!r} is already live")
        if not self._free_slots:
            return False
        slot = self._free_slots.pop()
        self._requests[rid] = _Request(slot, 0, {g: [] for g in range(self.n_groups)})
        self.fresh_slots.append(slot)
        return True

    def reserve(self, rid: Hashable, n_new: int) -> bool:
        """Pages for the next `n_new` positions in every group; all or nothing."""
        r = self._requests[rid]
        need = self.pages_needed(rid, n_new)
        if any(n > self.pools[g].n_free for g, n in enumerate(need)):
            return False
        for g, n in enumerate(need):
            r.pages[g].extend(self.pools[g].allocate(n))
        return True

    def commit(self, rid: Hashable, n_new: int) -> None:
        """`n_new` more positions are cached now.  A window group gives back every page that
        no later query can see: page j holds positions [j*ps, (j+1)*ps), the next query is at
        position >= tokens and sees keys > tokens - window."""
        r = self._requests[rid]
        if self.pages_for(r.tokens + n_new) > min((len(p) for p in r.pages.values()), default=1 << 60):
            raise PageError(f"request {rid!r}: commit of {n_new} tokens beyond its reserved pages")
        r.tokens += n_new
        for g, need in enumerate(self.group_needs):
            if need.window is None:
                continue
            first_visible = r.tokens - need.window + 1
            passed = max(0, first_visible // self.page_size)
            pages = r.pages[g]
            gone = [p for p in pages[:passed] if p != NO_PAGE]
            if gone:
                self.pools[g].release(gone)
                for j in range(min(passed, len(pages))):
                    pages[j] = NO_PAGE

    def release(self, rid: Hashable) -> None:
        """Gives back every page and the slot of a request that ended."""
        r = self._requests.pop(rid)
        for g, pages in r.pages.items():
            self.pools[g].release([p for p in pages if p != NO_PAGE])
        self._free_slots.append(r.slot)

    # ------------------------------------------------------------------ what kernels read
    def table_width(self, rids: Sequence[Hashable], group: int) -> int:
        return max((len(self._requests[r].pages[group]) for r in rids), default=0)

    def block_table(self, rids: Sequence[Hashable], group: int, width: Optional[int] = None) -> np.ndarray:
        """int32 [len(rids), width]: page id of logical page j of each request (NO_PAGE beyond
        its pages and for pages a window has passed)."""
        width = max(1, self.table_width(rids, group)) if width is None else width
        out = np.full((len(rids), width), NO_PAGE, dtype=np.int32)
        for i, rid in enumerate(rids):
            pages = self._requests[rid].pages[group]
            if len(pages) > width:
                raise ValueError(f"request {rid!r} holds {len(pages)} pages, table width is {width}")
            out[i, :len(pages)] = pages
        return out

    def take_fresh_slots(self) -> List[int]:
        out, self.fresh_slots = self.fresh_slots, []
        return out

    # ------------------------------------------------------------------ invariants (tests)
    def check(self) -> None:
        """No page lost, held twice or free while held; no slot shared."""
        for g, pool in enumerate(self.pools):
            owners: Dict[int, Hashable] = {}
            for rid, r in self._requests.items():
                for p in r.pages[g]:
                    if p == NO_PAGE:
                        continue
                    if p in owners:
                        raise PageError(f"group {g}: page {p} held by {owners[p]!r} and {rid!r}")
                    if not pool.is_held(p):
                        raise PageError(f"group {g}: page {p} of {rid!r} is on the free list")
                    owners[p] = rid
            if len(owners) != pool.n_held:
                raise PageError(f"group {g}: {pool.n_held} pages held, {len(owners)} owned: a page was lost")
            if len(set(pool._free)) != len(pool._free):
                raise PageError(f"group {g}: a page is on the free list twice")
        slots = [r.slot for r in self._requests.values()]
        if len(set(slots)) != len(slots) or set(slots) & set(self._free_slots):
            raise PageError("a slot is shared or free while held")
        if len(slots) + len(self._free_slots) != self.max_requests:
            raise PageError("a slot was lost")
