"""Device memory behind the cache manager: key and value pages of every cache group and the
arena of per-request state slots."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

import torch

from .manager import CacheManager
from .needs import StateNeed


@dataclass
class LayerCache:
    """What one layer's mixer sees of the cache during a step."""
    group: Optional[int]                        # cache group of the pages (None: no pages)
    kpages: Optional[torch.Tensor]              # [num_pages, kv_heads, page_size, head_dim]
    vpages: Optional[torch.Tensor]              # [num_pages, kv_heads, page_size, value head_dim]
    owns_pages: bool                            # False: reads another layer's pages, writes none
    states: Dict[str, torch.Tensor]             # name -> [slots, *shape] in the state's type (slot stride = arena row)


class DeviceCache:
    """Keys and values of a group are laid out [layer of group, page, kv head, slot in page, head_dim]
    (values with their own head size) in the cache dtype (the activation dtype of the run); every
    group has as many pages as its pool; a slot of the arena is a row of 4-byte words that holds the layers' states
    (float32 unless a mixer names another type).

    Behind the pool's pages every group holds one more page, and behind the requests' slots the arena
    one more slot, that the cache manager never hands out (`scratch_page`, `scratch_slot`): rows of a
    batch that stand for no request (the padding of a captured decode loop made for more rows than
    are live) write their keys, values and state there, where no request reads."""

    def __init__(self, manager: CacheManager, cache_dtype: torch.dtype, device: torch.device):
        self.manager = manager
        self.device = device
        self.cache_dtype = cache_dtype
        self.kpages: List[torch.Tensor] = []
        self.vpages: List[torch.Tensor] = []
        for g, need in enumerate(manager.group_needs):
            lead = (len(manager.group_layers[g]), manager.pools[g].num_pages + 1, need.kv_heads, manager.page_size)
            self.kpages.append(torch.zeros(lead + (need.head_dim,), dtype=cache_dtype, device=device))
            self.vpages.append(torch.zeros(lead + (need.value_dim,), dtype=cache_dtype, device=device))
        self.arena = torch.zeros((manager.max_requests + 1, max(1, manager.slot_floats)),
                                 dtype=torch.float32, device=device)
        self.scratch_slot = manager.max_requests
        self.scratch_page = [manager.pools[g].num_pages for g in range(len(manager.group_needs))]

    def nbytes(self) -> int:
        return sum(p.numel() * p.element_size() for p in self.kpages + self.vpages) + self.arena.numel() * 4

    def layer_view(self, layer: int, kv_source: Optional[int] = None) -> LayerCache:
        m = self.manager
        src = layer if kv_source is None else kv_source
        group = m.layer_group.get(src)
        k = v = None
        if group is not None:
            idx = m.group_layers[group].index(src)
            k, v = self.kpages[group][idx], self.vpages[group][idx]
        states = {}
        for (li, name), (off, shape, dtype) in m.state_layout.items():
            if li == layer:
                need = StateNeed(name, shape, dtype)
                words = self.arena[:, off:off + need.words]
                flat = words if dtype == "float32" else words.view(getattr(torch, dtype))[:, :need.numel]
                states[name] = flat.unflatten(1, shape) if shape else flat[:, 0]
        return LayerCache(group, k, v, kv_source is None and group is not None, states)

    def clear_fresh_slots(self) -> None:
        """Clears the state of slots that requests have taken since the last call."""
        for slot in self.manager.take_fresh_slots():
            self.arena[slot].zero_()
