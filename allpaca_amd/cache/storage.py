"""Device memory of the cache: one tensor per paged group and per state group,
allocated once.  A paged group's tensor is
[layers of the group, pages + 1, 2 (keys, values), kv_heads, page_tokens, head_dim];
inside a page, a key's elements lie together ([page_tokens, head_dim]) and a
value's positions lie together ([head_dim, page_tokens], the same count of
elements); the extra last page is never handed out (rows that pad a replayed
graph write there).  A state group's tensor is [layers of the group, slots + 1, *shape]."""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional

import torch

from .pages import CacheManager

_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16, "int32": torch.int32}


@dataclass
class PagedView:
    """What an attention-like mixer gets: its layer's pages and the step's block table of its group."""
    kv: torch.Tensor                 # [pages + 1, 2, kv_heads, page_tokens, head_dim]
    page_tokens: int
    window: Optional[int]
    writes: bool                     # False for a plan entry that borrows another entry's cache
    group: int
    block_table: Optional[torch.Tensor] = None   # set per step: int32 [segments, blocks]


@dataclass
class StateView:
    """What a mixer with state of its own gets: [slots + 1, *shape] and the step's slot of every segment."""
    state: torch.Tensor
    writes: bool
    group: int
    slots: Optional[torch.Tensor] = None         # set per step: int32 [segments]
    slots_host: Optional[List[int]] = None


class CacheStorage:
    def __init__(self, manager: CacheManager, kv_dtype: torch.dtype, device: torch.device):
        self.manager = manager
        self.device = device
        P = manager.page_tokens
        self.paged: List[torch.Tensor] = []
        for g in manager.paged_groups:
            shape = (len(g.entries), g.pool.num_pages + 1, 2, g.need.kv_heads, P, g.need.head_dim)
            self.paged.append(torch.zeros(shape, dtype=kv_dtype, device=device))
        self.state: List[torch.Tensor] = []
        for g in manager.state_groups:
            shape = (len(g.entries), manager.max_requests + 1, *g.need.shape)
            self.state.append(torch.zeros(shape, dtype=_DTYPES[g.need.dtype], device=device))

    def dummy_page(self, group: int) -> int:
        return self.manager.paged_groups[group].pool.num_pages

    def views(self, plan) -> list:
        """One view per plan entry (None for an entry without a cache)."""
        out = []
        for i, e in enumerate(plan):
            owner = i if e.cache_of is None else e.cache_of
            loc = self.manager.location.get(owner)
            if loc is None:
                out.append(None)
                continue
            kind, gi, li = loc
            if kind == "paged":
                need = self.manager.paged_groups[gi].need
                out.append(PagedView(self.paged[gi][li], self.manager.page_tokens, need.window, e.cache_of is None, gi))
            else:
                out.append(StateView(self.state[gi][li], e.cache_of is None, gi))
        return out

    def zero_slot(self, slot: int) -> None:
        for t in self.state:
            t[:, slot].zero_()

    def bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.paged + self.state)
