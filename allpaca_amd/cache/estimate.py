"""What the cache costs and how much of it fits: bytes of a page over all layers of its group, bytes of a state
slot, bytes for a number of tokens, tokens and pages for a number of bytes.  Pure arithmetic, no GPU.

The reference answers the same two questions for its own layout (`KvEstimate::bytes_for`, `tokens_for`:
crates/allpaca-core/src/engine.rs:8651-8680: bytes per token over the full-attention layers, plus bytes per token
over sliding-window layers that stop growing at the window) against a budget `kv.vram_bytes`."""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import List, Optional, Sequence

from ..parts.base import need_kind
from .pages import group_needs

_ELEM = {"float32": 4, "bfloat16": 2, "int32": 4}


@dataclass(frozen=True)
class GroupCost:
    page_bytes: int                  # one page over all layers of the group
    window: Optional[int]            # positions after which a request's pages of this group stop growing


@dataclass(frozen=True)
class CacheEstimate:
    page_tokens: int
    groups: List[GroupCost]
    slot_bytes: int                  # state of one request over all layers that keep state

    @staticmethod
    def of(needs: Sequence, page_tokens: int, cache_elem_bytes: int) -> "CacheEstimate":
        """`needs`: one cache need per plan entry (None for entries without a cache of their own);
        `cache_elem_bytes`: bytes of the run's cache element type, for needs that name none."""
        def elem(need) -> int:
            name = getattr(need, "dtype", None)
            return cache_elem_bytes if name is None else _ELEM[name]

        paged, state = group_needs(needs)
        groups = [GroupCost(len(entries) * math.prod(n.page_shape(page_tokens)) * elem(n), getattr(n, "window", None))
                  for n, entries in paged]
        slot = sum(len(entries) * math.prod(n.slot_shape()) * elem(n) for n, entries in state)
        return CacheEstimate(page_tokens, groups, slot)

    @property
    def bytes_per_page_of_every_group(self) -> int:
        """One more page in every group's pool (the pools have the same number of pages)."""
        return sum(g.page_bytes for g in self.groups)

    def pages_of_a_request(self, tokens: int, group: int) -> int:
        """Pages one request of `tokens` tokens holds in a group (a window's group stops growing; one page more
        than the window covers, since the window's ends fall inside pages)."""
        P = self.page_tokens
        w = self.groups[group].window
        n = -(-tokens // P)
        return n if w is None else min(n, -(-w // P) + 1)

    def bytes_for(self, tokens: int) -> int:
        """Cache bytes of one request that holds `tokens` tokens (pages are whole), without its state slot."""
        return sum(self.pages_of_a_request(tokens, g) * c.page_bytes for g, c in enumerate(self.groups))

    def tokens_for(self, nbytes: int) -> int:
        """Tokens of one request that fit `nbytes`: the largest count whose pages fit (2^40 if a request never
        outgrows the bytes: no group, or windows everywhere)."""
        lo, hi = 0, 1 << 40
        while lo < hi:
            mid = (lo + hi + 1) // 2
            if self.bytes_for(mid) <= nbytes:
                lo = mid
            else:
                hi = mid - 1
        return lo

    def pages_for_budget(self, nbytes: int, max_requests: int) -> int:
        """Pages of every group's pool when the cache may take `nbytes`: what is left after the state slots of
        `max_requests` requests (and the spare slot and page that padding rows use), in whole pages."""
        left = nbytes - (max_requests + 1) * self.slot_bytes
        per = self.bytes_per_page_of_every_group
        if per == 0:
            return 0
        return max(0, left // per - 1)
