"""Continuous batching: which requests run in the next step, and how many of
their tokens.  Pure bookkeeping over the cache manager; no GPU.

Every step, under a budget of `max_batch_tokens`:
 1. every running request that is decoding gets its one token;
 2. running requests still in their prompt get a portion (at most `chunk_tokens`,
    cut to what is left of the budget), oldest first;
 3. waiting requests are admitted in arrival order while fewer than
    `max_active_requests` run and pages for their first portion are free.
If the step's rows then come to a little more than a multiple of `row_tile` (the rows of a tile of the matrix
products: a step of 512 + 8 rows runs 5 tiles of 128 where 4 would nearly do, and its SwiGLU product takes 187 us
instead of 115), the last prompt portion is cut back to that multiple; the tokens left over go into a later portion.
A portion may have any size >= 1.  When a decoding request cannot get the page
its next token needs, the most recently admitted running request is preempted:
its pages go back, and it returns to the front of the waiting queue to be
recomputed from its prompt and the tokens it has generated.  The same happens
when no running request can advance at all (every one is in its prompt and waits
for a page that only another one's end would free): the most recently admitted
gives way until someone can go on, so some request advances in every step, the
one admitted first never loses what it has computed, and the engine cannot stall.  A request that could never fit the pool
is refused when it is added.

The reference advances one request per tick (`pick_runnable`, longest wait first,
crates/allpaca-core/src/scheduler.rs:607-664) by `prefill.chunk_tokens`
(crates/allpaca-core/src/engine.rs:4717-4756), batches only decode rows
(engine.rs:5451-5560), refuses admission above `engine.max_active_requests`
(engine.rs:3198-3200), takes a request's pages up front (engine.rs:3341-3349) and
so never runs out while decoding; what happens then is this engine's own rule."""
from __future__ import annotations

import ctypes
from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Dict, List, Optional, Tuple

from ..cache import CacheManager
from ..sampling.params import FinishReason, GenerationParams

WAITING, RUNNING, FINISHED = "waiting", "running", "finished"


class RequestTooLarge(ValueError):
    pass


@dataclass
class Request:
    id: int
    prompt: List[int]
    params: GenerationParams
    output: List[int] = field(default_factory=list)
    status: str = WAITING
    computed: int = 0                 # tokens whose keys and values are in the cache
    finish_reason: Optional[str] = None
    preemptions: int = 0
    order: int = 0                    # admission order (for the choice of a victim)
    # times (time.perf_counter): added, first scheduled, every token; the reference keeps a mean wait per poll and
    # counts of prefill and decode picks (crates/allpaca-core/src/engine.rs:3848-3872), here per request
    t_added: float = 0.0
    t_first_scheduled: Optional[float] = None
    t_tokens: List[float] = field(default_factory=list)

    def timing(self) -> dict:
        """Seconds: `queue` (added to first scheduled), `ttft` (added to first token), `itl` (mean time between
        tokens after the first); None where the event has not happened."""
        queue = None if self.t_first_scheduled is None else self.t_first_scheduled - self.t_added
        ttft = self.t_tokens[0] - self.t_added if self.t_tokens else None
        itl = ((self.t_tokens[-1] - self.t_tokens[0]) / (len(self.t_tokens) - 1)) if len(self.t_tokens) > 1 else None
        return {"queue": queue, "ttft": ttft, "itl": itl}

    @property
    def tokens(self) -> List[int]:
        return self.prompt + self.output

    @property
    def n_tokens(self) -> int:
        return len(self.prompt) + len(self.output)

    def token_slice(self, start: int, count: int) -> List[int]:
        """tokens[start : start + count] without building the whole list (a step asks for this every time)."""
        n = len(self.prompt)
        if start >= n:
            return self.output[start - n:start - n + count]
        if start + count <= n:
            return self.prompt[start:start + count]
        return self.prompt[start:] + self.output[:start + count - n]

    @property
    def left(self) -> int:
        """Tokens that must still run before the next token can be sampled."""
        return self.n_tokens - self.computed

    @property
    def decoding(self) -> bool:
        return self.left == 1 and len(self.output) > 0


@dataclass
class Scheduled:
    request: Request
    start: int                        # index of the first token of the portion in request.tokens
    count: int
    samples: bool                     # the portion reaches the end: the logits of its last row are wanted


@dataclass
class Plan:
    scheduled: List[Scheduled] = field(default_factory=list)
    preempted: List[Request] = field(default_factory=list)
    admitted: List[Request] = field(default_factory=list)

    @property
    def n_tokens(self) -> int:
        return sum(s.count for s in self.scheduled)


class Scheduler:
    """The face of the C++ scheduler (`csrc/host/sched.cpp`): it keeps the requests themselves (their tokens, their
    times) and mirrors what the C++ side decides into them (`status`, `computed`, `order`, `preemptions`) and into
    `waiting` and `running`, which hold the same requests in the same order as the queues there."""

    def __init__(self, cache: CacheManager, max_active_requests: int, max_batch_tokens: int, chunk_tokens: int,
                 row_tile: int = 0):
        from ..kernels import host
        self.cache = cache
        self.max_active = max_active_requests
        self.budget = max_batch_tokens
        self.chunk = chunk_tokens
        self.row_tile = row_tile          # 0: steps are not trimmed to whole tiles of rows
        self.waiting: Deque[Request] = deque()
        self.running: List[Request] = []
        self.preemption_count = 0
        self._lib = host.load()
        self._s = self._lib.apc_sched_new(cache.handle, max_active_requests, max_batch_tokens, chunk_tokens, row_tile)
        if not self._s:
            raise ValueError("the scheduler needs max_active_requests, max_batch_tokens and chunk_tokens above 0")
        self._by_cid: Dict[int, Request] = {}
        cap = max_active_requests + 8
        self._items = (ctypes.c_longlong * (4 * cap))()
        self._pre = (ctypes.c_longlong * cap)()
        self._adm = (ctypes.c_longlong * cap)()
        self._orders = (ctypes.c_int * cap)()
        self._n = (ctypes.c_int * 3)()
        self._cap = cap

    def __del__(self):
        if getattr(self, "_s", None):
            self._lib.apc_sched_free(self._s)
            self._s = None

    # ---- intake ----------------------------------------------------------------
    def add(self, req: Request) -> None:
        group = ctypes.c_int(0)
        worst = self._lib.apc_sched_too_large(self._s, len(req.prompt), req.params.max_tokens, ctypes.byref(group))
        if worst:
            raise RequestTooLarge(
                f"request {req.id}: {len(req.prompt)} prompt + {req.params.max_tokens} new tokens need {worst} "
                f"pages of {self.cache.page_tokens} positions, the whole pool has "
                f"{self.cache.paged_groups[group.value].pool.num_pages}")
        if not req.prompt:
            raise ValueError("a request needs at least one prompt token")
        req.status = WAITING
        req._cid = self.cache.new_id()      # its name in the cache manager's books, through every admission
        if self._lib.apc_sched_add(self._s, req._cid, len(req.prompt), len(req.output), req.params.max_tokens):
            raise ValueError(f"request {req.id} cannot be added")
        self._by_cid[req._cid] = req
        self.waiting.append(req)

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    # ---- one step's plan -------------------------------------------------------
    def plan(self) -> Plan:
        L = self._lib
        code = L.apc_sched_plan(self._s, self._items, self._cap, self._pre, self._adm, self._orders, self._cap, self._n)
        if code == -40:
            raise RequestTooLarge("a request cannot get a page although it runs alone")
        if code:
            raise RuntimeError(f"the scheduler failed with code {code}")
        n_sched, n_pre, n_adm = self._n[0], self._n[1], self._n[2]
        plan = Plan()
        for i in range(n_pre):       # in the order they gave way: each goes to the front of the queue
            victim = self._by_cid[self._pre[i]]
            self.cache.forget(victim.id)
            self.running.remove(victim)
            victim.status = WAITING
            victim.computed = 0
            victim.preemptions += 1
            self.preemption_count += 1
            self.waiting.appendleft(victim)
            plan.preempted.append(victim)
        for i in range(n_adm):       # from the front of the queue, in arrival order
            req = self.waiting.popleft()
            if req._cid != self._adm[i]:
                raise RuntimeError("the scheduler's queue and its mirror disagree")
            self.cache.remember(req.id, req._cid)
            req.status = RUNNING
            req.order = self._orders[i]
            self.running.append(req)
            plan.admitted.append(req)
        it = self._items
        for i in range(n_sched):
            plan.scheduled.append(Scheduled(self._by_cid[it[4 * i]], int(it[4 * i + 1]), int(it[4 * i + 2]),
                                            bool(it[4 * i + 3])))
        if n_pre:
            self.cache._tell_frees()
        return plan

    # ---- after the step ----------------------------------------------------------
    def advance(self, s: Scheduled) -> None:
        s.request.computed += s.count
        self._lib.apc_sched_advance(self._s, s.request._cid, s.count)

    def append_token(self, req: Request, token: int) -> Optional[str]:
        """Adds a sampled token; returns the finish reason if the request ends with it
        (stop id -> stop, `max_tokens` reached -> length; crates/allpaca-core/src/engine.rs:4607-4621)."""
        req.output.append(int(token))
        self._lib.apc_sched_token(self._s, req._cid)
        if int(token) in req.params.stop_token_ids:
            return FinishReason.STOP
        if len(req.output) >= req.params.max_tokens:
            return FinishReason.LENGTH
        return None

    def finish(self, req: Request, reason: str) -> None:
        """Pages and slot go back in the step that finishes the request."""
        req.status = FINISHED
        req.finish_reason = reason
        if req in self.running:
            self.running.remove(req)
        cid = getattr(req, "_cid", None)
        if cid is not None and cid in self._by_cid:
            del self._by_cid[cid]
            self._lib.apc_sched_finish(self._s, cid)       # releases what it holds in the cache
            self.cache.forget(req.id)
            self.cache._tell_frees()

    def abort(self, req: Request) -> None:
        if req in self.waiting:
            self.waiting.remove(req)
        self.finish(req, "abort")
