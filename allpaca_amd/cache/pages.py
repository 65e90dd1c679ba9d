"""Host-side bookkeeping of the cache: pools of pages, block tables, state slots.
No GPU is needed for any of it.

A model's plan entries are sorted into groups by what they need: entries whose
mixers ask for the same `PagedKV(kv_heads, head_dim, window)` share a group, a
group has a pool of pages of its own, and a request has one block table per
group (a page holds that group's layers for `page_tokens` positions).  Pages are
taken when a step needs them, given back when a request ends or when a window
has passed them, and handed out again (last freed, first reused).
Entries that ask for `FixedState` share a slot pool: one slot per request, taken
at admission and zeroed, given back at the end.  Every request gets a slot id
even if no layer keeps state.

The reference takes all pages of a request at admission and frees them when the
request handle drops (crates/allpaca-core/src/engine.rs:3341-3349, 409-432;
crates/allpaca-core/src/kv_tier.rs:341-532); recurrent layers get no pages
(crates/allpaca-core/src/model.rs:13392-13405)."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

from ..parts.base import CacheNeed, need_kind

FREED = -1  # block-table entry of a page that a window has passed


class CacheError(RuntimeError):
    pass


class OutOfPages(CacheError):
    pass


class OutOfSlots(CacheError):
    pass


class PagePool:
    """`num_pages` page ids handed out from a stack."""

    def __init__(self, num_pages: int):
        if num_pages <= 0:
            raise ValueError("a page pool needs at least one page")
        self.num_pages = num_pages
        self._free: List[int] = list(range(num_pages - 1, -1, -1))  # page 0 goes out first
        self._held = [False] * num_pages
        self.allocations = 0   # how many times a page was handed out (reuse shows as allocations > num_pages)
        self.on_free = None    # called with the id of every page that comes back (a debugging aid: see CacheStorage)

    @property
    def free_count(self) -> int:
        return len(self._free)

    def alloc(self) -> int:
        if not self._free:
            raise OutOfPages("no free page")
        p = self._free.pop()
        if self._held[p]:
            raise CacheError(f"page {p} was on the free list while held")
        self._held[p] = True
        self.allocations += 1
        return p

    def free(self, page: int) -> None:
        if not (0 <= page < self.num_pages):
            raise CacheError(f"page id {page} is outside the pool")
        if not self._held[page]:
            raise CacheError(f"page {page} freed twice")
        self._held[page] = False
        self._free.append(page)
        if self.on_free is not None:
            self.on_free(page)

    def held(self) -> List[int]:
        return [p for p, h in enumerate(self._held) if h]


class SlotPool(PagePool):
    """Slots for per-request state; same discipline as pages."""

    def alloc(self) -> int:
        try:
            return super().alloc()
        except OutOfPages:
            raise OutOfSlots("no free state slot") from None


@dataclass
class PagedGroup:
    need: CacheNeed                    # kind "pages"
    entries: List[int]                 # plan entries stored in this group, in order
    pool: PagePool


@dataclass
class StateGroup:
    need: CacheNeed                    # kind "slot"
    entries: List[int]


@dataclass
class _Sequence:
    slot: int
    length: int = 0                    # positions committed
    reserved: int = 0                  # positions that pages exist for
    tables: List[List[int]] = field(default_factory=list)   # per paged group: page ids, FREED where a window passed
    version: int = 0                   # changes whenever an entry of a table was taken away or replaced


def group_needs(needs: Sequence[CacheNeed]) -> Tuple[List[Tuple[CacheNeed, List[int]]], List[Tuple[CacheNeed, List[int]]]]:
    """Plan entries sorted by what they need: ([(need of kind "pages", entries)], [(need of kind "slot", entries)]).
    Equal needs share a group; a need is any object with the members `parts.base` lists."""
    paged: Dict[CacheNeed, List[int]] = {}
    state: Dict[CacheNeed, List[int]] = {}
    for i, n in enumerate(needs):
        try:
            kind = need_kind(n)
        except TypeError as e:
            raise TypeError(f"plan entry {i}: {e}") from None
        if kind == "pages":
            paged.setdefault(n, []).append(i)
        elif kind == "slot":
            state.setdefault(n, []).append(i)
    return list(paged.items()), list(state.items())


class CacheManager:
    """Block tables and slots for live requests.

    `num_pages`: pages of every paged group's pool (an int for all, or one per group)."""

    def __init__(self, needs: Sequence[CacheNeed], page_tokens: int, num_pages, max_requests: int):
        if page_tokens <= 0:
            raise ValueError("page_tokens must be positive")
        self.page_tokens = page_tokens
        paged, state = group_needs(needs)
        if isinstance(num_pages, int):
            num_pages = [num_pages] * len(paged)
        if len(num_pages) != len(paged):
            raise ValueError(f"{len(paged)} paged groups but {len(num_pages)} pool sizes")
        self.paged_groups = [PagedGroup(n, e, PagePool(np_)) for (n, e), np_ in zip(paged, num_pages)]
        self.state_groups = [StateGroup(n, e) for n, e in state]
        self.slots = SlotPool(max_requests)
        self.max_requests = max_requests
        self._seqs: Dict[Hashable, _Sequence] = {}
        self._versions = 0
        # plan entry -> ("paged", group index, index inside the group) | ("state", ...) ; filled for owners only
        self.location: Dict[int, Tuple[str, int, int]] = {}
        for gi, g in enumerate(self.paged_groups):
            for li, e in enumerate(g.entries):
                self.location[e] = ("paged", gi, li)
        for gi, g in enumerate(self.state_groups):
            for li, e in enumerate(g.entries):
                self.location[e] = ("state", gi, li)

    # ---- requests ------------------------------------------------------------
    def __contains__(self, seq) -> bool:
        return seq in self._seqs

    def live(self) -> List[Hashable]:
        return list(self._seqs)

    def admit(self, seq) -> int:
        """Registers a request and gives it a state slot (the caller zeroes the slot's state)."""
        if seq in self._seqs:
            raise CacheError(f"request {seq!r} is already live")
        slot = self.slots.alloc()
        self._versions += 1
        self._seqs[seq] = _Sequence(slot, tables=[[] for _ in self.paged_groups], version=self._versions)
        return slot

    def slot_of(self, seq) -> int:
        return self._seqs[seq].slot

    def length(self, seq) -> int:
        return self._seqs[seq].length

    def _first_needed(self, need: CacheNeed, next_pos: int) -> int:
        """First position whose page a row at `next_pos` or later can still read."""
        window = getattr(need, "window", None)
        if window is None:
            return 0
        return max(0, next_pos - window + 1)

    def pages_needed(self, seq, n_new: int) -> List[int]:
        """Pages each group must still take so that positions up to length + n_new exist."""
        s = self._seqs[seq]
        end = s.length + n_new
        want = -(-end // self.page_tokens)
        return [max(0, want - len(t)) for t in s.tables]

    def can_reserve(self, seq, n_new: int, spare: Optional[List[int]] = None) -> bool:
        """`spare`: pages per group already promised to others in the same step."""
        need = self.pages_needed(seq, n_new)
        spare = spare or [0] * len(need)
        return all(n + sp <= g.pool.free_count for n, sp, g in zip(need, spare, self.paged_groups))

    def reserve(self, seq, n_new: int) -> None:
        """Takes the pages for the next `n_new` positions, in every group or in none."""
        s = self._seqs[seq]
        need = self.pages_needed(seq, n_new)
        for n, g in zip(need, self.paged_groups):
            if n > g.pool.free_count:
                raise OutOfPages(f"request {seq!r} needs {n} more pages, the pool has {g.pool.free_count} free")
        for n, g, t in zip(need, self.paged_groups, s.tables):
            for _ in range(n):
                t.append(g.pool.alloc())
        s.reserved = max(s.reserved, s.length + n_new)

    def commit(self, seq, n_new: int) -> None:
        """The step wrote `n_new` positions; pages that every later row's window has passed go back."""
        s = self._seqs[seq]
        if s.length + n_new > s.reserved:
            raise CacheError(f"request {seq!r}: commit of {n_new} positions beyond what was reserved")
        s.length += n_new
        for g, t in zip(self.paged_groups, s.tables):
            first = self._first_needed(g.need, s.length)
            for i in range(min(first // self.page_tokens, len(t))):
                if t[i] != FREED:
                    g.pool.free(t[i])
                    t[i] = FREED
                    self._versions += 1
                    s.version = self._versions

    def truncate(self, seq, length: int) -> None:
        """Forgets positions >= length (pages wholly beyond go back).  Not possible below a window's edge."""
        s = self._seqs[seq]
        if length > s.length:
            raise CacheError("truncate beyond the current length")
        keep = -(-length // self.page_tokens)
        for g, t in zip(self.paged_groups, s.tables):
            if any(p == FREED for p in t[self._first_needed(g.need, length) // self.page_tokens:keep]):
                raise CacheError("truncate below pages that a window has already given back")
            while len(t) > keep:
                p = t.pop()
                self._versions += 1
                s.version = self._versions
                if p != FREED:
                    g.pool.free(p)
        s.length = length
        s.reserved = min(s.reserved, keep * self.page_tokens)

    def release(self, seq) -> None:
        s = self._seqs.pop(seq)
        for g, t in zip(self.paged_groups, s.tables):
            for p in t:
                if p != FREED:
                    g.pool.free(p)
        self.slots.free(s.slot)

    def block_table(self, seq, group: int) -> List[int]:
        return self._seqs[seq].tables[group]

    def table_version(self, seq) -> int:
        """A number that is the same as at an earlier call only if the request's block tables have only grown since
        (no page taken away or replaced, and it is the same admission of the request)."""
        return self._seqs[seq].version

    def free_pages(self, group: int = 0) -> int:
        return self.paged_groups[group].pool.free_count

    def pages_for_tokens(self, n_tokens: int) -> int:
        return -(-n_tokens // self.page_tokens)

    # ---- self-check (tests) ----------------------------------------------------
    def check(self) -> None:
        """No page lost, none held twice, free + held = pool."""
        for gi, g in enumerate(self.paged_groups):
            seen: Dict[int, Hashable] = {}
            for sid, s in self._seqs.items():
                for p in s.tables[gi]:
                    if p == FREED:
                        continue
                    if p in seen:
                        raise CacheError(f"group {gi}: page {p} held by {seen[p]!r} and {sid!r}")
                    seen[p] = sid
            held = set(g.pool.held())
            if held != set(seen):
                raise CacheError(f"group {gi}: pool holds {sorted(held)}, block tables hold {sorted(seen)}")
            if len(held) + g.pool.free_count != g.pool.num_pages:
                raise CacheError(f"group {gi}: {len(held)} held + {g.pool.free_count} free != {g.pool.num_pages}")
        slots = [s.slot for s in self._seqs.values()]
        if len(set(slots)) != len(slots) or set(slots) != set(self.slots.held()):
            raise CacheError("state slots and live requests disagree")
