"""Device memory of the cache: one tensor per paged group and per state group,
allocated once.  A paged group's tensor is [layers of the group, pages + 1,
*need.page_shape(page_tokens)] (for keys and values: [2, kv_heads, page_tokens,
head_dim]; inside a page a key's elements lie together and a value's positions
lie together, the same count of elements); the extra last page is never handed
out (rows that pad a replayed graph write there).  A state group's tensor is
[layers of the group, slots + 1, *need.slot_shape()].  The element type is the
need's own, or the run's cache type where the need names none."""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import List, Optional

import torch

from .pages import CacheError, CacheManager

_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16, "int32": torch.int32}


@dataclass
class PagedView:
    """What an attention-like mixer gets: its layer's pages and the step's block table of its group."""
    kv: torch.Tensor                 # [pages + 1, *need.page_shape(page_tokens)]; keys and values: [.., 2, kv_heads, page_tokens, head_dim]
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


class CacheTooLarge(CacheError):
    pass


class CacheStorage:
    def __init__(self, manager: CacheManager, kv_dtype: torch.dtype, device: torch.device):
        self.manager = manager
        self.device = device
        P = manager.page_tokens

        def dtype_of(need) -> torch.dtype:
            name = getattr(need, "dtype", None)
            if name is None:
                return kv_dtype
            if name not in _DTYPES:
                raise CacheError(f"cache need {need!r}: element type {name!r} is not one of {sorted(_DTYPES)}")
            return _DTYPES[name]

        def nbytes(shape, dt) -> int:
            return math.prod(shape) * torch.empty((), dtype=dt).element_size()

        paged = [((len(g.entries), g.pool.num_pages + 1, *g.need.page_shape(P)), dtype_of(g.need))
                 for g in manager.paged_groups]
        state = [((len(g.entries), manager.max_requests + 1, *g.need.slot_shape()), dtype_of(g.need))
                 for g in manager.state_groups]
        need = sum(nbytes(sh, dt) for sh, dt in paged + state)
        if device.type == "cuda":
            free, _ = torch.cuda.mem_get_info(device)
            free += torch.cuda.memory_reserved(device) - torch.cuda.memory_allocated(device)  # held by torch, unused
            if need > free:
                per_page = sum(nbytes(sh, dt) // sh[1] for sh, dt in paged)
                raise CacheTooLarge(
                    f"the cache needs {need / 2**30:.1f} GiB ({[sh[1] - 1 for sh, _ in paged]} pages of {P} tokens, "
                    f"{per_page / 2**20:.2f} MiB a page over all layers) but {free / 2**30:.1f} GiB of device memory "
                    f"are free: ask for fewer pages (max_tokens / num_pages)")
        self.paged: List[torch.Tensor] = [torch.zeros(sh, dtype=dt, device=device) for sh, dt in paged]
        self.state: List[torch.Tensor] = [torch.zeros(sh, dtype=dt, device=device) for sh, dt in state]

    def poison_free_pages(self, value: float = 1e30) -> None:
        """A debugging aid against stale reads: every page that is free, now and whenever one comes back, is filled
        with `value`, so that a key or value read from a page that the request has not written itself shows in the
        logits at once.  The default is large and finite; with NaN even a stale value that is multiplied by a weight
        of 0 shows (no kernel may let one into a product)."""
        for t, g in zip(self.paged, self.manager.paged_groups):
            held = set(g.pool.held())
            for page in range(g.pool.num_pages):
                if page not in held:
                    t[:, page].fill_(value)
            g.pool.on_free = lambda page, t=t: t[:, page].fill_(value)

    def dummy_page(self, group: int) -> int:
        return self.manager.paged_groups[group].pool.num_pages

    def views(self, plan) -> list:
        """One view per plan entry (None for an entry without a cache)."""
        def view(loc, writes: bool):
            kind, gi, li = loc
            if kind == "paged":
                need = self.manager.paged_groups[gi].need
                return PagedView(self.paged[gi][li], self.manager.page_tokens, getattr(need, "window", None), writes, gi)
            return StateView(self.state[gi][li], writes, gi)

        out = []
        for i, e in enumerate(plan):
            owner = i if e.cache_of is None else e.cache_of
            loc = self.manager.location.get(owner)
            if loc is not None:
                out.append(view(loc, e.cache_of is None))
                continue
            # several parts of the entry keep a cache: a dict role -> view
            roles = {k[1]: v for k, v in self.manager.location.items() if isinstance(k, tuple) and k[0] == owner}
            out.append({role: view(loc, e.cache_of is None) for role, loc in roles.items()} or None)
        return out

    def zero_slot(self, slot: int) -> None:
        for t in self.state:
            t[:, slot].zero_()

    def bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.paged + self.state)
