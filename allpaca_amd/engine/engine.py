"""The engine: requests in, tokens out.  It owns the model, the step function,
the scheduler and the sampler, and offers the reference's calls
(`generate`, `generate_stream`, `begin_request`, `step`/`poll`:
crates/allpaca-core/src/engine.rs:2895, 3002, 3167, 3650, 3661)."""
from __future__ import annotations

import os
import shutil
import sys
import tempfile
import time
from typing import Dict, Iterator, List, Mapping, Optional, Sequence

import torch

from ..config import EngineConfig
from ..models import load_model
from ..sampling.params import FinishReason, GenerationOutput, GenerationParams, TokenEvent
from ..sampling.sampler import Sampler
from .batch import Entry
from .runner import ModelRunner
from .scheduler import FINISHED, RUNNING, Request, Scheduled, Scheduler

_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32}


class _AheadStep:
    """A decode step that already runs on the GPU, model and sampling, fed with the tokens of the step before on the
    GPU itself; the host has not seen either step's tokens yet.  `dead`: requests that ended (a stop token, an
    abort) after it was queued: their rows are ignored."""

    def __init__(self, scheduled, pending):
        self.scheduled, self.pending, self.dead = scheduled, pending, set()


class Engine:
    def __init__(self, model: str, config: Optional[EngineConfig] = None, **options):
        """`model`: a folder with config.json and model.safetensors.  Options are those of `EngineConfig`."""
        cfg = config or EngineConfig()
        for k, v in options.items():
            if not hasattr(cfg, k):
                raise TypeError(f"unknown engine option {k!r}")
            setattr(cfg, k, v)
        cfg.validate()
        if not torch.cuda.is_available():
            raise RuntimeError("no GPU is visible; the engine has no CPU path")
        # positions the tables are made for: what the pool can hold if its size is given, else the model's own limit
        positions = cfg.num_pages * cfg.page_tokens or cfg.max_tokens or None
        model_config, bound = load_model(model, _DTYPES[cfg.dtype], cfg.device, max_positions=positions)
        self._assemble(model_config, bound, cfg)

    def _assemble(self, model_config, model, cfg: EngineConfig) -> None:
        """Runner, scheduler and sampler around a model that is bound to its weights."""
        self.config, self.model_config, self.model = cfg, model_config, model
        num_pages = cfg.num_pages or -(-cfg.max_tokens // cfg.page_tokens) or self.pages_that_fit(model, cfg)
        self.runner = ModelRunner(model, cfg.page_tokens, num_pages, cfg.max_active_requests, use_graphs=cfg.use_graphs)
        self.scheduler = Scheduler(self.runner.cache, cfg.max_active_requests, cfg.max_batch_tokens, cfg.chunk_tokens,
                                   row_tile=cfg.step_row_tile if cfg.dtype == "bfloat16" else 0)
        self.sampler = Sampler(self.runner.rt.device, cfg.seed)
        self.requests: Dict[int, Request] = {}
        self._ahead: Optional[_AheadStep] = None
        self._next_id = 0
        # counters (the reference's: prefill chunks, forwards, batched rows, pages in use,
        # crates/allpaca-core/src/engine.rs:4656-4679, 5099-5101, 5644-5649)
        self.stats = {"steps": 0, "prefill_tokens": 0, "decode_tokens": 0, "preemptions": 0, "prefill_portions": 0,
                      "batched_rows": 0, "graph_replays": 0, "pages_in_use": 0, "pages_in_use_peak": 0}
        # the logits that tokens are chosen from, kept for whoever asks (`tap_logits`), appended to a file
        # (ALLPACA_LOGITS_DUMP=<file>) or their two largest printed (ALLPACA_LOGIT_TRACE=1)
        self._tap: Optional[list] = None
        self._dump_path = os.environ.get("ALLPACA_LOGITS_DUMP") or None
        self._trace_top2 = os.environ.get("ALLPACA_LOGIT_TRACE") == "1"

    @staticmethod
    def pages_that_fit(model, cfg: EngineConfig) -> int:
        """Pages of the pool when neither `num_pages` nor `max_tokens` is given: floor((budget - state slots) / bytes
        of a page over all layers), the budget being `kv_bytes` or the device memory that is free now (the weights
        are loaded) minus `kv_reserve_bytes`; at most what `max_active_requests` requests of the longest context
        need."""
        from ..cache import CacheEstimate, CacheTooLarge
        rt = model.rt
        est = CacheEstimate.of(model.cache_needs(), cfg.page_tokens, torch.empty((), dtype=rt.dtype).element_size())
        budget = cfg.kv_bytes
        if not budget:
            free, _ = torch.cuda.mem_get_info(rt.device)
            free += torch.cuda.memory_reserved(rt.device) - torch.cuda.memory_allocated(rt.device)
            budget = free - (cfg.kv_reserve_bytes or Engine.reserve_bytes(model, cfg))
        pages = est.pages_for_budget(budget, cfg.max_active_requests)
        most = cfg.max_active_requests * -(-rt.max_positions // cfg.page_tokens)
        pages = min(pages, most)
        if pages <= 0:
            raise CacheTooLarge(f"no page of the cache fits: the budget is {budget / 2**30:.2f} GiB "
                                f"(kv_bytes, or free device memory less kv_reserve_bytes), a page over all layers takes "
                                f"{est.bytes_per_page_of_every_group / 2**20:.2f} MiB")
        return pages

    @staticmethod
    def reserve_bytes(model, cfg: EngineConfig) -> int:
        """Device memory kept out of the cache pool when it is sized from what is free: a step's work space (the
        residual stream and the widest layer's outputs for `max_batch_tokens` rows, in 32-bit terms and twice over for
        partial sums of products with K in slices), the logits of two decode steps under way and the sampler's scratch
        for `max_active_requests` rows, and 1 GiB for graphs, pinned staging and the allocator's slack."""
        spec = model.spec
        widest = max([sum(ps.shape[0] for ps in b.param_specs().values() if len(ps.shape) == 2 and ps.store == "compute")
                      for b in model.blocks] or [0])
        step = cfg.max_batch_tokens * (4 * spec.hidden_size + 4 * widest) * 2
        out = cfg.max_active_requests * (3 * 4 * spec.vocab_size + (256 << 10))
        return step + out + (1 << 30)

    @classmethod
    def from_model(cls, model_config, model, config: EngineConfig) -> "Engine":
        """An engine around a `DecoderModel` that the caller has built and bound to weights on the GPU (weights made
        in place, without a model folder)."""
        config.validate()
        eng = cls.__new__(cls)
        eng._assemble(model_config, model, config)
        return eng

    @classmethod
    def synthetic(cls, config_json: Mapping, seed: int = 0, config: Optional[EngineConfig] = None, **options) -> "Engine":
        """An engine on random weights: the model folder is written to a temporary place first and removed once
        the weights are on the GPU (the reference's `--synthetic`, crates/allpaca-core/src/engine.rs:1577-1586)."""
        from ..weights import write_model_folder
        dtype = _DTYPES[(config.dtype if config else options.get("dtype", EngineConfig().dtype))]
        folder = tempfile.mkdtemp(prefix="allpaca_amd_synthetic_")
        try:
            write_model_folder(folder, config_json, seed, dtype, keep_tensors=False)
            return cls(folder, config, **options)
        finally:
            shutil.rmtree(folder, ignore_errors=True)

    # ---- requests ------------------------------------------------------------
    def warm_up(self, max_context: Optional[int] = None) -> int:
        """Captures the decode graphs of every batch size up to `max_active_requests` and every context bucket up to
        `max_context` (default: the longest the run allows) before serving starts; returns their number."""
        return self.runner.capture_decode_graphs(self.config.max_active_requests, max_context)

    def add_request(self, prompt_token_ids: Sequence[int], params: Optional[GenerationParams] = None) -> int:
        params = params or GenerationParams()
        prompt = [int(t) for t in prompt_token_ids]
        for t in prompt:
            if not (0 <= t < self.runner.vocab_size):
                raise ValueError(f"token {t} is outside the vocabulary of {self.runner.vocab_size}")
        if len(prompt) + params.max_tokens > self.runner.rt.max_positions:
            raise ValueError(f"{len(prompt)} prompt + {params.max_tokens} new tokens exceed the "
                             f"{self.runner.rt.max_positions} positions this engine was set up for")
        rid = self._next_id
        self._next_id += 1
        req = Request(rid, prompt, params, t_added=time.perf_counter())
        self.scheduler.add(req)
        self.requests[rid] = req
        return rid

    begin_request = add_request

    def abort(self, request_id: int) -> None:
        if self._ahead is not None:
            self._ahead.dead.add(request_id)
        req = self.requests.pop(request_id, None)
        if req is not None and req.status != FINISHED:
            self.scheduler.abort(req)

    def has_unfinished(self) -> bool:
        return self.scheduler.has_work()

    # ---- the logits behind the tokens ----------------------------------------------------------------------
    def tap_logits(self, on: bool = True) -> None:
        """Keep a copy of the logits every sampled token is chosen from (or stop and drop them), so that two runs'
        distributions can be compared (the reference's `tap_logits`, crates/allpaca-core/src/engine.rs:1179-1183).
        While it is on, every step waits for its logits to reach the host."""
        self._tap = [] if on else None

    def take_tapped_logits(self) -> List[tuple]:
        """The logits tapped since the last call, in the order the tokens were chosen: (request id, index of the
        generated token in its request, float32 array [vocab]) each (crates/allpaca-core/src/engine.rs:1185-1189)."""
        out, self._tap = (self._tap or []), ([] if self._tap is not None else None)
        return out

    def _observe_logits(self, logits, sampled, extra: int) -> None:
        """The tap, the dump file and the trace of the two largest logits (crates/allpaca-core/src/sampling.rs:84-127:
        `ALLPACA_LOGIT_TRACE`, `ALLPACA_LOGITS_DUMP`, a vocabulary per sampled token as little-endian float32)."""
        rows = logits[:len(sampled)].float().cpu().numpy()
        for s, row in zip(sampled, rows):
            if self._tap is not None:
                self._tap.append((s.request.id, len(s.request.output) + extra, row.copy()))
            if self._trace_top2:
                top = row.argsort()[-2:][::-1] if row.size > 1 else [0, 0]
                print(f"logit_trace {int(top[0])} {row[top[0]]:.6f} {int(top[1])} {row[top[1]]:.6f}", file=sys.stderr)
        if self._dump_path:
            try:
                with open(self._dump_path, "ab") as f:
                    f.write(rows.astype("<f4").tobytes())
            except OSError as e:
                print(f"ALLPACA_LOGITS_DUMP: cannot write {self._dump_path}: {e}", file=sys.stderr)
                self._dump_path = None

    # ---- one tick ---------------------------------------------------------------
    def step(self) -> List[TokenEvent]:
        """One batch through the model: every decoding request advances by a token, prompts by a portion.
        While nothing but decoding goes on, the step after this one is queued on the GPU before this one's tokens
        have reached the host (`_launch_ahead`): the GPU goes from step to step without waiting for the host, and
        the host reads each step's tokens while the next one runs."""
        ahead, self._ahead = self._ahead, None
        if ahead is not None:
            scheduled = [s for s in ahead.scheduled if s.request.id not in ahead.dead]
            sampled_all, pending = ahead.scheduled, ahead.pending
        else:
            plan = self.scheduler.plan()
            self.stats["preemptions"] += len(plan.preempted)
            for req in plan.admitted:
                self.runner.storage.zero_slot(self.runner.cache.slot_of(req.id))
            if not plan.scheduled:
                return []
            scheduled = plan.scheduled
            now = time.perf_counter()
            entries = []
            for s in scheduled:
                if s.request.t_first_scheduled is None:
                    s.request.t_first_scheduled = now
                toks = s.request.token_slice(s.start, s.count)
                entries.append(Entry(s.request.id, toks, [s.count - 1] if s.samples else []))
            logits = self.runner.step(entries)
            sampled_all = [s for s in scheduled if s.samples]
            pending = self._launch_sampling(logits, sampled_all, 0) if sampled_all else None
        st = self.stats
        for s in scheduled:
            self.scheduler.advance(s)
            decode = bool(s.request.output) and s.count == 1
            st["decode_tokens" if decode else "prefill_tokens"] += s.count
            st["prefill_portions"] += 0 if decode else 1
            st["batched_rows"] += s.count
        st["steps"] += 1
        cache = self.runner.cache
        st["pages_in_use_peak"] = max(st["pages_in_use_peak"],
                                      sum(g.pool.num_pages - g.pool.free_count for g in cache.paged_groups))
        events: List[TokenEvent] = []
        if pending is not None:
            if ahead is None or not ahead.dead:
                self._ahead = self._launch_ahead(scheduled, sampled_all, pending)
            tokens = pending.wait()
            now = time.perf_counter()       # the token ids are on the host: the step is over
            for s, tok in zip(sampled_all, tokens):
                if ahead is not None and s.request.id in ahead.dead:
                    continue
                s.request.t_tokens.append(now)
                reason = self.scheduler.append_token(s.request, tok)
                events.append(TokenEvent(s.request.id, int(tok), reason, len(s.request.prompt)))
                if reason is not None:
                    self.scheduler.finish(s.request, reason)
                    if self._ahead is not None:
                        self._ahead.dead.add(s.request.id)    # its row of the queued step counts for nothing
            if self._ahead is not None and all(s.request.id in self._ahead.dead for s in self._ahead.scheduled):
                self._ahead = None
        st["graph_replays"] = self.runner.graph_replays
        st["pages_in_use"] = sum(g.pool.num_pages - g.pool.free_count for g in cache.paged_groups)
        return events

    def _launch_sampling(self, logits, sampled, extra: int):
        """Queues the choice of a token for every row; `extra`: tokens of each request that are on their way and
        not appended yet (they count for the index of the random number)."""
        if self._tap is not None or self._dump_path or self._trace_top2:
            self._observe_logits(logits, sampled, extra)
        return self.sampler.launch(logits, [s.request.params for s in sampled],
                                   [len(s.request.output) + extra for s in sampled])

    def _launch_ahead(self, scheduled, sampled, pending) -> Optional["_AheadStep"]:
        """If the next step is sure to be one more token for exactly the requests of this one (nothing waits, every
        running request samples a token in this step, in the order decode steps have, and none reaches its
        `max_tokens` with it), it is queued now: pages reserved, positions and tables filled in, the tokens copied
        from this step's sampling result on the GPU, model and sampling launched.  A request that ends with this
        step's token (a stop id) has a row in the queued step that is ignored; its pages go back as always, and
        whatever later gets them is queued behind that row's write."""
        sch = self.scheduler
        if sch.waiting or len(scheduled) != len(sch.running) or len(sampled) != len(scheduled):
            return None
        for s in scheduled:
            r = s.request
            if not s.samples or r.status != RUNNING or len(r.output) + 1 >= r.params.max_tokens:
                return None
        order = sorted((s.request for s in scheduled), key=lambda r: r.order)   # as the scheduler orders decodes
        if [r.id for r in order] != [s.request.id for s in sampled]:
            return None     # the sampled rows lie in another order (a prompt ended in this step): the next step will do
        handle = self.runner.prepare_decode([r.id for r in order])
        if handle is None:
            return None
        logits = self.runner.run_fed(handle, pending.device)
        nxt = [Scheduled(r, r.computed, 1, True) for r in order]
        return _AheadStep(nxt, self._launch_sampling(logits, nxt, 1))

    poll = step

    # ---- whole generations ---------------------------------------------------------
    def generate_stream(self, prompt_token_ids: Sequence[int],
                        params: Optional[GenerationParams] = None) -> Iterator[TokenEvent]:
        rid = self.add_request(prompt_token_ids, params)
        while self.requests[rid].status != FINISHED:
            for ev in self.step():
                if ev.request_id == rid:
                    yield ev
        self.requests.pop(rid, None)

    def generate(self, prompts: Sequence[Sequence[int]], params=None) -> List[GenerationOutput]:
        """Runs all prompts to the end under continuous batching; `params` is one `GenerationParams`
        for all or one per prompt."""
        if params is None or isinstance(params, GenerationParams):
            params = [params] * len(prompts)
        ids = [self.add_request(p, q) for p, q in zip(prompts, params)]
        while any(self.requests[i].status != FINISHED for i in ids):
            self.step()
        out = []
        for i in ids:
            r = self.requests.pop(i)
            out.append(GenerationOutput(list(r.output), len(r.prompt), len(r.output), r.finish_reason, r.timing()))
        return out
