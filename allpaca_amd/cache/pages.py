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

import ctypes
from dataclasses import dataclass
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

from ..parts.base import CacheNeed, need_kind

FREED = -1  # block-table entry of a page that a window has passed


class CacheError(RuntimeError):
    pass


class OutOfPages(CacheError):
    pass


class OutOfSlots(CacheError):
    pass


def _host():
    from ..kernels import host
    return host.load()


_POOL_ERRORS = {-22: OutOfPages, -27: CacheError, -28: CacheError, -29: CacheError}


def _raise_pool(code: int, page=None):
    if code == -22:
        raise OutOfPages("no free page")
    if code == -27:
        raise CacheError(f"page id {page} is outside the pool")
    if code == -28:
        raise CacheError(f"page {page} freed twice")
    if code == -29:
        raise CacheError("a page was on the free list while held")
    raise CacheError(f"page pool: error {code}")


class PagePool:
    """`num_pages` page ids handed out from a stack (the books are kept in `csrc/host/cache.cpp`)."""

    def __init__(self, num_pages: int, _borrowed=None, _owner=None):
        if num_pages <= 0:
            raise ValueError("a page pool needs at least one page")
        self._lib = _host()
        self._owner = _owner             # the cache manager whose pool this is (keeps it alive), or None
        self._p = _borrowed if _borrowed is not None else self._lib.apc_pool_new(num_pages)
        self.num_pages = num_pages
        self._on_free = None

    def __del__(self):
        if getattr(self, "_owner", None) is None and getattr(self, "_p", None):
            self._lib.apc_pool_free(self._p)
            self._p = None

    @property
    def on_free(self):
        """Called with the id of every page that comes back (a debugging aid: see CacheStorage)."""
        return self._on_free

    @on_free.setter
    def on_free(self, fn) -> None:
        self._on_free = fn
        self._lib.apc_pool_log_frees(self._p, 1 if fn is not None else 0)

    def _tell_frees(self) -> None:
        if self._on_free is None:
            return
        buf = (ctypes.c_int * 256)()
        while True:
            k = self._lib.apc_pool_drain(self._p, buf, 256)
            for i in range(k):
                self._on_free(buf[i])
            if k < 256:
                return

    @property
    def free_count(self) -> int:
        return self._lib.apc_pool_free_count(self._p)

    @property
    def allocations(self) -> int:
        """How many times a page was handed out (reuse shows as allocations > num_pages)."""
        return self._lib.apc_pool_allocations(self._p)

    def alloc(self) -> int:
        p = self._lib.apc_pool_alloc(self._p)
        if p < 0:
            _raise_pool(p)
        return p

    def free(self, page: int) -> None:
        code = self._lib.apc_pool_give_back(self._p, int(page))
        if code:
            _raise_pool(code, page)
        self._tell_frees()

    def held(self) -> List[int]:
        buf = (ctypes.c_int * self.num_pages)()
        k = self._lib.apc_pool_held(self._p, buf, self.num_pages)
        return list(buf[:k])


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


def group_needs(needs: Sequence[CacheNeed]) -> Tuple[List[Tuple[CacheNeed, List[int]]], List[Tuple[CacheNeed, List[int]]]]:
    """Plan entries sorted by what they need: ([(need of kind "pages", entries)], [(need of kind "slot", entries)]).
    Equal needs share a group; a need is any object with the members `parts.base` lists."""
    paged: Dict[CacheNeed, list] = {}
    state: Dict[CacheNeed, list] = {}
    for i, asked in enumerate(needs):
        # one need of the entry, or a dict role -> need: its parts are then stored under (entry, role)
        for key, n in ([((i, role), n) for role, n in asked.items()] if isinstance(asked, dict) else [(i, asked)]):
            try:
                kind = need_kind(n)
            except TypeError as e:
                raise TypeError(f"plan entry {i}: {e}") from None
            if kind == "pages":
                paged.setdefault(n, []).append(key)
            elif kind == "slot":
                state.setdefault(n, []).append(key)
    return list(paged.items()), list(state.items())


class CacheManager:
    """Block tables and slots for live requests.

    `num_pages`: pages of every paged group's pool (an int for all, or one per group).  Requests are named by any
    hashable; the books themselves are kept in C++ (`csrc/host/cache.cpp`) under ids that this class hands out, so
    that the step packer and the scheduler there read them without coming back to Python."""

    def __init__(self, needs: Sequence[CacheNeed], page_tokens: int, num_pages, max_requests: int):
        if page_tokens <= 0:
            raise ValueError("page_tokens must be positive")
        self.page_tokens = page_tokens
        paged, state = group_needs(needs)
        if isinstance(num_pages, int):
            num_pages = [num_pages] * len(paged)
        if len(num_pages) != len(paged):
            raise ValueError(f"{len(paged)} paged groups but {len(num_pages)} pool sizes")
        if len(paged) > 8:
            raise ValueError(f"{len(paged)} paged groups: the cache manager keeps books for at most 8")
        if any(n <= 0 for n in num_pages) or max_requests <= 0:
            raise ValueError("a page pool needs at least one page")
        self._lib = L = _host()
        windows = [(-1 if getattr(n, "window", None) is None else int(n.window)) for n, _ in paged]
        G = len(paged)
        self._c = L.apc_cache_new(page_tokens, G, (ctypes.c_int * max(G, 1))(*windows),
                                  (ctypes.c_int * max(G, 1))(*[int(n) for n in num_pages]), max_requests)
        if not self._c:
            raise ValueError("the cache manager could not be set up with these sizes")
        self.paged_groups = [PagedGroup(n, e, PagePool(np_, L.apc_cache_pool(self._c, gi), self))
                             for gi, ((n, e), np_) in enumerate(zip(paged, num_pages))]
        self.state_groups = [StateGroup(n, e) for n, e in state]
        self.slots = SlotPool(max_requests, L.apc_cache_pool(self._c, -1), self)
        self.max_requests = max_requests
        self._ids: Dict[Hashable, int] = {}
        self._next_id = 0
        self._need = (ctypes.c_int * 8)()
        self._table = (ctypes.c_int * 64)()
        # plan entry -> ("paged", group index, index inside the group) | ("state", ...) ; filled for owners only
        self.location: Dict[int, Tuple[str, int, int]] = {}
        for gi, g in enumerate(self.paged_groups):
            for li, e in enumerate(g.entries):
                self.location[e] = ("paged", gi, li)
        for gi, g in enumerate(self.state_groups):
            for li, e in enumerate(g.entries):
                self.location[e] = ("state", gi, li)

    def __del__(self):
        if getattr(self, "_c", None):
            self._lib.apc_cache_free(self._c)
            self._c = None

    @property
    def handle(self):
        """The books' address, for the C++ step packer and scheduler."""
        return self._c

    def id_of(self, seq) -> int:
        """The id under which the C++ side knows a live request."""
        return self._ids[seq]

    # The C++ scheduler admits and releases requests in the books itself; it tells this face afterwards.
    def new_id(self) -> int:
        """An id that no request has had: for a request that the C++ scheduler will admit under it."""
        self._next_id += 1
        return self._next_id - 1

    def remember(self, seq, sid: int) -> None:
        """`seq` was admitted in the books under id `sid`."""
        if seq in self._ids:
            raise CacheError(f"request {seq!r} is already live")
        self._ids[seq] = sid

    def forget(self, seq) -> None:
        """`seq` was released in the books."""
        self._ids.pop(seq, None)

    def _fail(self, code: int, seq, what: str = ""):
        if code == -20:
            raise CacheError(f"request {seq!r} is already live")
        if code == -21:
            raise OutOfSlots("no free state slot")
        if code == -22:
            raise OutOfPages(f"request {seq!r} needs more pages than the pool has free{what}")
        if code == -23:
            raise CacheError(f"request {seq!r}: commit of positions beyond what was reserved")
        if code == -24:
            raise CacheError("truncate beyond the current length")
        if code == -25:
            raise CacheError("truncate below pages that a window has already given back")
        if code == -26:
            raise KeyError(seq)
        if code == -28:
            raise CacheError("a page was freed twice")
        raise CacheError(f"cache manager: error {code}")

    def _tell_frees(self) -> None:
        for g in self.paged_groups:
            if g.pool._on_free is not None:
                g.pool._tell_frees()

    # ---- requests ------------------------------------------------------------
    def __contains__(self, seq) -> bool:
        return seq in self._ids

    def live(self) -> List[Hashable]:
        return list(self._ids)

    def admit(self, seq) -> int:
        """Registers a request and gives it a state slot (the caller zeroes the slot's state)."""
        if seq in self._ids:
            raise CacheError(f"request {seq!r} is already live")
        sid = self._next_id
        slot = self._lib.apc_cache_admit(self._c, sid)
        if slot < 0:
            self._fail(slot, seq)
        self._next_id += 1
        self._ids[seq] = sid
        return slot

    def slot_of(self, seq) -> int:
        return self._lib.apc_cache_slot(self._c, self._ids[seq])

    def length(self, seq) -> int:
        return self._lib.apc_cache_length(self._c, self._ids[seq])

    def pages_needed(self, seq, n_new: int) -> List[int]:
        """Pages each group must still take so that positions up to length + n_new exist."""
        self._lib.apc_cache_pages_needed(self._c, self._ids[seq], int(n_new), self._need)
        return list(self._need[:len(self.paged_groups)])

    def can_reserve(self, seq, n_new: int, spare: Optional[List[int]] = None) -> bool:
        """`spare`: pages per group already promised to others in the same step."""
        need = self.pages_needed(seq, n_new)
        spare = spare or [0] * len(need)
        return all(n + sp <= g.pool.free_count for n, sp, g in zip(need, spare, self.paged_groups))

    def reserve(self, seq, n_new: int) -> None:
        """Takes the pages for the next `n_new` positions, in every group or in none."""
        code = self._lib.apc_cache_reserve(self._c, self._ids[seq], int(n_new))
        if code:
            what = ""
            if code == -22:
                what = f" ({self.pages_needed(seq, n_new)} wanted, {[g.pool.free_count for g in self.paged_groups]} free)"
            self._fail(code, seq, what)

    def commit(self, seq, n_new: int) -> None:
        """The step wrote `n_new` positions; pages that every later row's window has passed go back."""
        code = self._lib.apc_cache_commit(self._c, self._ids[seq], int(n_new))
        if code:
            self._fail(code, seq)
        self._tell_frees()

    def truncate(self, seq, length: int) -> None:
        """Forgets positions >= length (pages wholly beyond go back).  Not possible below a window's edge."""
        code = self._lib.apc_cache_truncate(self._c, self._ids[seq], int(length))
        if code:
            self._fail(code, seq)
        self._tell_frees()

    def release(self, seq) -> None:
        sid = self._ids.pop(seq)
        code = self._lib.apc_cache_release(self._c, sid)
        self._tell_frees()
        if code:
            self._fail(code, seq)

    def block_table(self, seq, group: int) -> List[int]:
        sid = self._ids[seq]
        n = self._lib.apc_cache_table(self._c, sid, group, self._table, len(self._table))
        if n > len(self._table):
            self._table = (ctypes.c_int * (2 * n))()
            n = self._lib.apc_cache_table(self._c, sid, group, self._table, len(self._table))
        if n < 0:
            self._fail(n, seq)
        return list(self._table[:n])

    def table_version(self, seq) -> int:
        """A number that is the same as at an earlier call only if the request's block tables have only grown since
        (no page taken away or replaced, and it is the same admission of the request)."""
        return self._lib.apc_cache_version(self._c, self._ids[seq])

    def free_pages(self, group: int = 0) -> int:
        return self.paged_groups[group].pool.free_count

    def pages_for_tokens(self, n_tokens: int) -> int:
        return -(-n_tokens // self.page_tokens)

    # ---- self-check (tests) ----------------------------------------------------
    def check(self) -> None:
        """No page lost, none held twice, free + held = pool."""
        if self._lib.apc_cache_check(self._c):
            raise CacheError(self._lib.apc_cache_why(self._c).decode())
