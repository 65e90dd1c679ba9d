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
    def __init__(self, cache: CacheManager, max_active_requests: int, max_batch_tokens: int, chunk_tokens: int,
                 row_tile: int = 0):
        self.cache = cache
        self.max_active = max_active_requests
        self.budget = max_batch_tokens
        self.chunk = chunk_tokens
        self.row_tile = row_tile          # 0: steps are not trimmed to whole tiles of rows
        self.waiting: Deque[Request] = deque()
        self.running: List[Request] = []
        self._admissions = 0
        self.preemption_count = 0

    # ---- intake ----------------------------------------------------------------
    def add(self, req: Request) -> None:
        need = self.cache.pages_for_tokens(len(req.prompt) + req.params.max_tokens)
        for g in self.cache.paged_groups:
            window = getattr(g.need, "window", None)
            window_pages = None if window is None else self.cache.pages_for_tokens(window) + 1
            worst = need if window_pages is None else min(need, window_pages + self.cache.pages_for_tokens(self.chunk))
            if worst > g.pool.num_pages:
                raise RequestTooLarge(
                    f"request {req.id}: {len(req.prompt)} prompt + {req.params.max_tokens} new tokens need {worst} "
                    f"pages of {self.cache.page_tokens} positions, the whole pool has {g.pool.num_pages}")
        if not req.prompt:
            raise ValueError("a request needs at least one prompt token")
        req.status = WAITING
        self.waiting.append(req)

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    # ---- one step's plan -------------------------------------------------------
    def _fits(self, req: Request, n: int, promised: List[int]) -> bool:
        need = self.cache.pages_needed(req.id, n)
        return all(need[g] + promised[g] <= self.cache.free_pages(g) for g in range(len(need)))

    def _promise(self, req: Request, n: int, promised: List[int]) -> None:
        for g, k in enumerate(self.cache.pages_needed(req.id, n)):
            promised[g] += k

    def _preempt(self, victim: Request, plan: Plan) -> None:
        self.cache.release(victim.id)
        self.running.remove(victim)
        victim.status = WAITING
        victim.computed = 0
        victim.preemptions += 1
        self.preemption_count += 1
        self.waiting.appendleft(victim)
        plan.preempted.append(victim)

    def plan(self) -> Plan:
        plan = self._plan_once(Plan())
        while not plan.scheduled and len(self.running) > 1:
            # Nobody can advance: the requests in their prompts hold all pages between them.  The newest gives its
            # pages back (it is not admitted again in this step), until the oldest can go on.
            self._preempt(max(self.running, key=lambda r: r.order), plan)
            plan = self._plan_once(plan)
        return plan

    def _plan_once(self, plan: Plan) -> Plan:
        """Fills `plan.scheduled` (from nothing); what `plan` lists as preempted and admitted so far stays."""
        plan.scheduled = []
        budget = self.budget
        promised = [0] * len(self.cache.paged_groups)
        # 1. decodes, oldest admission first.  If a page is missing, the newest running request that is not
        #    yet part of this step gives way, be it the asking request itself.
        for req in sorted([r for r in self.running if r.decoding], key=lambda r: r.order):
            if req.status != RUNNING or budget <= 0:
                continue
            while req.status == RUNNING and not self._fits(req, 1, promised):
                victims = [r for r in self.running if all(s.request is not r for s in plan.scheduled)]
                if victims == [req] and len(self.running) == 1:
                    raise RequestTooLarge(f"request {req.id} cannot get a page although it runs alone")
                self._preempt(max(victims, key=lambda r: r.order), plan)
            if req.status != RUNNING:
                continue
            self._promise(req, 1, promised)
            plan.scheduled.append(Scheduled(req, req.computed, 1, True))
            budget -= 1
        # 2. portions of prompts that are under way
        for req in sorted([r for r in self.running if not r.decoding], key=lambda r: r.order):
            if budget <= 0:
                break
            if req.status != RUNNING:
                continue
            n = min(req.left, self.chunk, budget)
            while n > 0 and not self._fits(req, n, promised):
                n = self._shrink(req, n, promised)
            if n <= 0:
                continue
            self._promise(req, n, promised)
            plan.scheduled.append(Scheduled(req, req.computed, n, n == req.left))
            budget -= n
        # 3. admissions, in arrival order; the first that does not fit blocks the ones behind it
        while self.waiting and budget > 0 and len(self.running) < self.max_active:
            req = self.waiting[0]
            if req in plan.preempted:
                break  # it was just preempted for lack of pages; it comes back in a later step
            slot_ok = self.cache.slots.free_count > 0
            if not slot_ok:
                break
            self.cache.admit(req.id)
            n = min(req.left, self.chunk, budget)
            while n > 0 and not self._fits(req, n, promised):
                n = self._shrink(req, n, promised)
            if n <= 0:
                self.cache.release(req.id)
                break
            self.waiting.popleft()
            req.status = RUNNING
            self._admissions += 1
            req.order = self._admissions
            self.running.append(req)
            plan.admitted.append(req)
            self._promise(req, n, promised)
            plan.scheduled.append(Scheduled(req, req.computed, n, n == req.left))
            budget -= n
        self._trim_to_tiles(plan)
        return plan

    def _trim_to_tiles(self, plan: Plan) -> None:
        """Cuts the last prompt portion back when the step's rows overshoot a multiple of `row_tile` by up to a quarter
        of a tile (two tiles or more remain, and at least half of the portion)."""
        if not self.row_tile:
            return
        total = sum(s.count for s in plan.scheduled)
        over = total % self.row_tile
        if total < 2 * self.row_tile or not 0 < over <= self.row_tile // 4:
            return
        for s in reversed(plan.scheduled):
            if not s.request.decoding and 2 * (s.count - over) >= s.count:
                s.count -= over
                s.samples = False
                return

    def _shrink(self, req: Request, n: int, promised: List[int]) -> int:
        """The largest portion below n that the free pages allow (0 if none)."""
        P = self.cache.page_tokens
        room = min(self.cache.free_pages(g) - promised[g] for g in range(len(promised))) if promised else 0
        have = min((len(self.cache.block_table(req.id, g)) for g in range(len(promised))), default=0)
        can = (have + max(room, 0)) * P - self.cache.length(req.id)
        return max(0, min(n - 1, can))

    # ---- after the step ----------------------------------------------------------
    def advance(self, s: Scheduled) -> None:
        s.request.computed += s.count

    def append_token(self, req: Request, token: int) -> Optional[str]:
        """Adds a sampled token; returns the finish reason if the request ends with it
        (stop id -> stop, `max_tokens` reached -> length; crates/allpaca-core/src/engine.rs:4607-4621)."""
        req.output.append(int(token))
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
        if req.id in self.cache:
            self.cache.release(req.id)

    def abort(self, req: Request) -> None:
        if req in self.waiting:
            self.waiting.remove(req)
        self.finish(req, "abort")
