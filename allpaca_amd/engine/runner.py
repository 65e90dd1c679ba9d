"""The step function: a batch of (request, its next tokens) in, logits at the
wanted places out.  It runs only the tokens it is given, as one batch, against
the cache that earlier steps left; portions of prompts stand beside single
decoded tokens, cut anywhere.

The reference has three forwards (one token, one sequence's rows, many
sequences' rows: crates/allpaca-core/src/model.rs:8195, 8894, 8839) and never
mixes a prompt portion with decode rows in one of them
(crates/allpaca-core/src/engine.rs:5451-5607); this is the one generalisation."""
from __future__ import annotations

import ctypes
import gc
import os
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..cache import CacheManager, CacheStorage, OutOfPages, PagedView, StateView
from ..models.decoder import DecoderModel
from .batch import Entry, StepInfo, StepLayout, pack_step


class StepError(ValueError):
    pass


class ModelRunner:
    def __init__(self, model: DecoderModel, page_tokens: int, num_pages, max_requests: int,
                 kv_dtype: Optional[torch.dtype] = None, use_graphs: bool = False, poison_free_pages=False):
        if model.rt is None:
            raise StepError("the model has no weights bound")
        self.model = model
        self.rt = model.rt
        self.cache = CacheManager(model.cache_needs(), page_tokens, num_pages, max_requests)
        self.storage = CacheStorage(self.cache, kv_dtype or self.rt.dtype, self.rt.device)
        # a debugging aid: True fills free pages with 1e30, a number (NaN too) with that number
        if poison_free_pages is not False and poison_free_pages is not None and poison_free_pages != 0:
            self.storage.poison_free_pages(1e30 if poison_free_pages is True else float(poison_free_pages))
        elif os.environ.get("ALLPACA_POISON_FREE_PAGES") == "1":
            self.storage.poison_free_pages()
        self.views = self.storage.views(model.spec.plan)
        # The model's steps from C++ (one call a step, intermediates in a work space) if every part of it describes
        # itself to the executor; else, or with ALLPACA_AMD_PYTHON_WALK=1, the parts are walked in Python.
        self.native = None
        if os.environ.get("ALLPACA_AMD_PYTHON_WALK") != "1":
            from .native import NativeProgram
            self.native = NativeProgram.of(model, self.views)
        self.pad_pages = [self.storage.dummy_page(g) for g in range(len(self.cache.paged_groups))]
        self.vocab_size = model.spec.vocab_size
        # decode-only steps are replayed as HIP graphs when every part of the model allows it: a single part that
        # plans on the host (a feed-forward that gathers rows per expert, say) would be replayed with a stale plan
        parts = [model.embedding, model.final_norm, model.head] + [p for b in model.blocks for p in b.parts.values()]
        self.use_graphs = bool(use_graphs) and all(getattr(p, "graph_safe", False) for p in parts)
        from ..kernels import ops
        if self.rt.dtype == torch.bfloat16 and not ops.FORCE_PLAIN:
            from ..kernels import tuned
            tuned.check_chip(self.rt.device)
        self.tile_rows = ops.attention_tile_rows(self.rt.dtype)          # how the attention kernel wants longer segments cut
        self.position_axes = int(getattr(model.spec, "position_axes", 1))
        self.graphs: Dict[Tuple[int, int], "DecodeGraph"] = {}
        self.graph_replays = 0
        self.steps = 0
        # The C++ side of a step (csrc/host/pack.cpp): entries checked against the cache's books, pages taken, the
        # description written into one of a few pinned buffers that take turns (a buffer is written again only when
        # the copy out of it has run).
        from ..kernels import host as _host
        self._host, self._hostlib = _host, _host.load()
        self._staging: List[list] = []        # [pinned tensor, its numpy view, event of the last copy out of it]
        self._staging_at = 0
        self._pad_pages = np.asarray(self.pad_pages or [0], dtype=np.int32)
        self._finding = _host.ApcStepFinding()
        self._packed = _host.ApcPacked()

    # ---- requests ------------------------------------------------------------
    def admit(self, seq: Hashable) -> int:
        slot = self.cache.admit(seq)
        self.storage.zero_slot(slot)
        return slot

    def release(self, seq: Hashable) -> None:
        self.cache.release(seq)

    def length(self, seq: Hashable) -> int:
        return self.cache.length(seq)

    # ---- a step ----------------------------------------------------------------
    def validate(self, entries: Sequence[Entry]) -> None:
        seen = set()
        for e in entries:
            if e.seq in seen:
                raise StepError(f"request {e.seq!r} appears twice in one step")
            seen.add(e.seq)
            if e.seq not in self.cache:
                raise StepError(f"request {e.seq!r} is not admitted")
            n = len(e.tokens)
            if n == 0:
                raise StepError(f"request {e.seq!r} brings no tokens")
            for t in e.tokens:
                if not (0 <= int(t) < self.vocab_size):  # crates/allpaca-core/src/model.rs:8215-8219
                    raise StepError(f"request {e.seq!r}: token {t} is outside the vocabulary of {self.vocab_size}")
            for w in e.want:
                if not (0 <= int(w) < n):
                    raise StepError(f"request {e.seq!r}: wanted place {w} is outside its {n} tokens")
            if self.cache.length(e.seq) + n > self.rt.max_positions:
                raise StepError(f"request {e.seq!r}: position {self.cache.length(e.seq) + n - 1} is beyond the "
                                f"{self.rt.max_positions} positions this run was set up for")

    # ---- a step through the C++ packer ---------------------------------------------------------------------
    def _flatten(self, entries: Sequence[Entry]):
        """The entries as arrays for the C++ side: (ids, tokens a request, all tokens, wanted places a request, all
        wanted places).  Requests named twice or not admitted are refused here, where their names are known."""
        ids, n_tok, toks, n_want, wants = [], [], [], [], []
        known = self.cache._ids
        seen = set()
        for e in entries:
            if e.seq in seen:
                raise StepError(f"request {e.seq!r} appears twice in one step")
            seen.add(e.seq)
            sid = known.get(e.seq)
            if sid is None:
                raise StepError(f"request {e.seq!r} is not admitted")
            ids.append(sid)
            n_tok.append(len(e.tokens))
            toks.extend(e.tokens)
            n_want.append(len(e.want))
            wants.extend(e.want)
        t64 = np.asarray(toks, dtype=np.int64)
        if t64.size and (int(t64.min()) < 0 or int(t64.max()) >= self.vocab_size):   # (also what int32 cannot hold)
            at = int(np.flatnonzero((t64 < 0) | (t64 >= self.vocab_size))[0])
            e = entries[int(np.searchsorted(np.cumsum(n_tok), at, side="right"))]
            raise StepError(f"request {e.seq!r}: token {int(t64[at])} is outside the vocabulary of {self.vocab_size}")
        w64 = np.asarray(wants, dtype=np.int64)
        if w64.size and (int(w64.min()) < 0 or int(w64.max()) >= (1 << 31) - 1):
            w64 = np.clip(w64, -1, (1 << 31) - 2)       # refused below, with its request's name
        return (np.asarray(ids, dtype=np.int64), np.asarray(n_tok, dtype=np.int32), t64.astype(np.int32),
                np.asarray(n_want, dtype=np.int32), w64.astype(np.int32))

    def _prepare(self, entries: Sequence[Entry], flat) -> None:
        """Checks the step and takes its pages, for all requests or for none."""
        ids, n_tok, toks, n_want, wants = flat
        f = self._finding
        code = self._hostlib.apc_step_prepare(self.cache.handle, self.vocab_size, self.rt.max_positions, len(entries),
                                              ids.ctypes.data, n_tok.ctypes.data, toks.ctypes.data, n_want.ctypes.data,
                                              wants.ctypes.data, ctypes.byref(f))
        if code == 0:
            return
        if code < 0:
            self.cache._fail(code, None)
        e = entries[f.entry] if f.what != 7 else None
        if f.what == 3:
            raise StepError(f"request {e.seq!r} brings no tokens")
        if f.what == 4:
            raise StepError(f"request {e.seq!r}: token {f.value} is outside the vocabulary of {self.vocab_size}")
        if f.what == 5:
            raise StepError(f"request {e.seq!r}: wanted place {f.value} is outside its {len(e.tokens)} tokens")
        if f.what == 6:
            raise StepError(f"request {e.seq!r}: position {f.value} is beyond the {self.rt.max_positions} positions "
                            f"this run was set up for")
        if f.what == 7:
            raise OutOfPages(f"the step needs {f.value} new pages in group {f.entry}, {f.extra} are free")
        raise StepError(f"the step was refused (finding {f.what} at entry {f.entry})")

    def _staging_buffer(self, ints: int):
        """A pinned buffer of at least `ints` int32 that no copy is reading any more."""
        if len(self._staging) < 4:
            t = torch.zeros(max(ints, 1 << 14), dtype=torch.int32).pin_memory()
            self._staging.append([t, t.numpy(), None])
            slot = self._staging[-1]
        else:
            slot = self._staging[self._staging_at]
            self._staging_at = (self._staging_at + 1) % len(self._staging)
            if slot[2] is not None:
                slot[2].synchronize()
            if slot[0].numel() < ints:
                slot[0] = torch.zeros(max(ints, 2 * slot[0].numel()), dtype=torch.int32).pin_memory()
                slot[1] = slot[0].numpy()
        return slot

    def _pack_flat(self, entries: Sequence[Entry], flat) -> StepInfo:
        ids, n_tok, toks, n_want, wants = flat
        L, c, p = self._hostlib, self.cache.handle, self._packed
        n = len(entries)
        L.apc_pack_layout(c, n, ids.ctypes.data, n_tok.ctypes.data, n_want.ctypes.data, self.tile_rows, 1, ctypes.byref(p))
        slot = self._staging_buffer(p.total)
        host, view = slot[0], slot[1]
        code = L.apc_pack_step(c, n, ids.ctypes.data, n_tok.ctypes.data, toks.ctypes.data, n_want.ctypes.data,
                               wants.ctypes.data, self.tile_rows, 1, self._pad_pages.ctypes.data, view.ctypes.data,
                               view.size, ctypes.byref(p))
        if code:
            self._host.check(code, "packing a step")
        dev = torch.empty(p.total, dtype=torch.int32, device=self.rt.device)
        dev.copy_(host[:p.total], non_blocking=True)
        if slot[2] is None:
            slot[2] = torch.cuda.Event()
        slot[2].record()
        lay = StepLayout(p.T, p.S, p.R, p.n_decode, p.n_tiles, 1, list(p.table_width[:p.n_groups]))
        o = p.off
        return lay.info(dev, view[o[3]:o[3] + n].tolist(), n_tok.tolist(), view[o[5]:o[5] + n].tolist(),
                        view[o[6]:o[6] + n].tolist(), p.max_decode_context, p.n_decode == p.T)

    def step(self, entries: Sequence[Entry]) -> Optional[torch.Tensor]:
        """Runs one batch; returns float32 logits [sum of wanted places, vocab] (device), or None."""
        if not entries:
            return None
        if self.position_axes == 1 and all(e.positions is None for e in entries):
            flat = self._flatten(entries)
            self._prepare(entries, flat)
            if self.use_graphs and all(len(e.tokens) == 1 and list(e.want) == [0] for e in entries):
                logits = self.graph_step(entries)
            else:
                logits = self.forward(self._pack_flat(entries, flat))
            code = self._hostlib.apc_step_commit(self.cache.handle, len(entries), flat[0].ctypes.data, flat[1].ctypes.data)
            if code:
                self.cache._fail(code, None)
            self.cache._tell_frees()
            self.steps += 1
            return logits
        # positions on more than one axis: the step is packed in Python
        self.validate(entries)
        # pages for this step's tokens only, for all requests or for none
        need = [0] * len(self.cache.paged_groups)
        for e in entries:
            for g, n in enumerate(self.cache.pages_needed(e.seq, len(e.tokens))):
                need[g] += n
        for g, n in enumerate(need):
            if n > self.cache.free_pages(g):
                raise OutOfPages(f"the step needs {n} new pages in group {g}, {self.cache.free_pages(g)} are free")
        for e in entries:
            self.cache.reserve(e.seq, len(e.tokens))
        if self.use_graphs and all(len(e.tokens) == 1 and list(e.want) == [0] and e.positions is None for e in entries):
            logits = self.graph_step(entries)
        else:
            logits = self.forward(self.pack(entries))
        for e in entries:
            self.cache.commit(e.seq, len(e.tokens))
        self.steps += 1
        return logits

    def pack(self, entries: Sequence[Entry]) -> StepInfo:
        pos0 = [self.cache.length(e.seq) for e in entries]
        slots = [self.cache.slot_of(e.seq) for e in entries]
        tables = [[self.cache.block_table(e.seq, g) for e in entries] for g in range(len(self.cache.paged_groups))]
        return pack_step(entries, pos0, slots, tables, self.rt.device, self.pad_pages, tile_rows=self.tile_rows,
                         position_axes=self.position_axes)

    def forward(self, info: StepInfo) -> Optional[torch.Tensor]:
        """The model on a packed step: logits at the wanted rows."""
        if self.native is not None:
            return self.native.forward(info)
        return self.model.forward(info, self.bind_views(info))

    def bind_views(self, info: StepInfo) -> list:
        for entry in self.views:
            for v in (entry.values() if isinstance(entry, dict) else (entry,)):
                if isinstance(v, PagedView):
                    v.block_table = info.block_tables[v.group]
                elif isinstance(v, StateView):
                    v.slots = info.state_slots
                    v.slots_host = info.host_slots
        return self.views

    # ---- decode-only steps as HIP graphs -----------------------------------------------
    def graph_step(self, entries: Sequence[Entry]) -> torch.Tensor:
        """A step in which every request brings one token and wants its logits: the launches of the whole
        model are replayed from a graph captured for (rows rounded up, see `_row_bucket`, context rounded
        up to a power of two); only the batch description is copied in."""
        seqs = [e.seq for e in entries]
        g = self._graph_for(seqs)
        g.fill(seqs)
        return self._launch(g, [e.tokens[0] for e in entries])

    def _bucket(self, n: int, longest: int) -> tuple:
        """(rows, span) of the graph for n requests of which the longest will hold `longest` tokens."""
        rows = self._row_bucket(n)
        span = max(256, 1 << (longest - 1).bit_length())
        span = min(span, -(-self.rt.max_positions // self.cache.page_tokens) * self.cache.page_tokens)
        return rows, max(span, longest)

    @staticmethod
    def _row_bucket(n: int) -> int:
        """Rows of the graph that takes n requests: the next power of two, but every even number from 8 to 16: there the
        products stream the weights through one 16-row MFMA tile and read, beside every weight tile, the activations of
        the rows that exist (padding rows are rows of their own), so a step of 9 rows in a graph of 16 took 4.36 ms at
        8B shapes where 10 rows take about what 8 do (3.6 ms)."""
        if 8 < n <= 16:
            return (n + 1) // 2 * 2
        return 1 << max(0, (n - 1).bit_length())

    def _graph_for(self, seqs: Sequence[Hashable]) -> "DecodeGraph":
        key = self._bucket(len(seqs), max(self.cache.length(s) for s in seqs) + 1)
        g = self.graphs.get(key)
        if g is None:
            g = self.graphs[key] = DecodeGraph(self, *key)
        return g

    def capture_decode_graphs(self, max_rows: int, max_context: Optional[int] = None) -> int:
        """Captures now, instead of at its first use (some tens of milliseconds in the middle of serving), the
        graph of every bucket that decode steps of up to `max_rows` requests and `max_context` tokens (default:
        the run's limit) can ask for.  Returns how many graphs were captured."""
        if not self.use_graphs:
            return 0
        top = min(max_context or self.rt.max_positions, self.rt.max_positions)
        keys = set()
        for n in sorted({self._row_bucket(k) for k in range(1, max_rows + 1)}):
            longest = 1
            while True:
                keys.add(self._bucket(min(n, max_rows), min(longest, top)))
                if longest >= top:
                    break
                longest *= 2
        made = 0
        for key in sorted(keys):
            if key not in self.graphs:
                self.graphs[key] = DecodeGraph(self, *key)
                made += 1
        return made

    def _launch(self, g: "DecodeGraph", tokens: Sequence[int]) -> torch.Tensor:
        g.set_tokens(tokens)
        g.upload()
        g.replay()
        self.graph_replays += 1
        return g.logits[:len(tokens)]

    # A decode-only step in two halves, so that the host can do the first half while the GPU still works on the step
    # before and the tokens are not known yet.
    def prepare_decode(self, seqs: Sequence[Hashable]) -> Optional["PreparedDecode"]:
        """Everything of a step of one token per request that does not need the tokens: pages taken, the graph
        chosen, positions and block tables written into its description.  None if this step cannot be prepared
        (no graphs, no page free, a position beyond the run's limit): the caller then goes the ordinary way, which
        says what is wrong.  What was reserved stays reserved for its request."""
        if not self.use_graphs or not seqs:
            return None
        need = [0] * len(self.cache.paged_groups)
        for s in seqs:
            if s not in self.cache or self.cache.length(s) + 1 > self.rt.max_positions:
                return None
            for gi, k in enumerate(self.cache.pages_needed(s, 1)):
                need[gi] += k
        if any(k > self.cache.free_pages(gi) for gi, k in enumerate(need)):
            return None
        for s in seqs:
            self.cache.reserve(s, 1)
        g = self._graph_for(seqs)
        g.fill(seqs)
        return PreparedDecode(g, list(seqs))

    def run_fed(self, prepared: "PreparedDecode", device_tokens: torch.Tensor) -> torch.Tensor:
        """The second half: the tokens go in, the step runs; nothing may have happened to the requests since
        `prepare_decode`.  The tokens are still on the GPU (int32, one per request, in the order of the
        prepared requests: what the sampling kernel of the step before wrote).  They are copied into the step's
        description on the GPU, so the step can be queued before the host has seen them."""
        g, n = prepared.graph, len(prepared.seqs)
        if device_tokens.dtype != torch.int32 or device_tokens.numel() < n or device_tokens.device != g.dev.device:
            raise StepError("tokens fed on the GPU must be int32, one per prepared request, on the engine's device")
        g.upload()
        g.layout.part(g.dev, "tokens")[:n].copy_(device_tokens[:n])
        g.replay()
        self.graph_replays += 1
        for s in prepared.seqs:
            self.cache.commit(s, 1)
        self.steps += 1
        return g.logits[:n]


class PreparedDecode:
    def __init__(self, graph: "DecodeGraph", seqs: List[Hashable]):
        self.graph, self.seqs = graph, seqs


HEAD_ENTRIES = 2   # plan entries in the first of a decode step's two graphs


class DecodeGraph:
    """The launches of one decode step for `rows` single-token requests whose contexts fit `span` positions.
    Rows beyond the live requests are padding: token 0 at position 0 of the spare page and the spare slot."""

    def __init__(self, runner: ModelRunner, rows: int, span: int):
        self.runner, self.rows, self.span = runner, rows, span
        cache = runner.cache
        self.widths = [-(-span // cache.page_tokens) for _ in cache.paged_groups]
        # the description is laid out as every step's is (`StepLayout`): one row, one segment and one wanted row per
        # request
        self.layout = lay = StepLayout(rows, rows, rows, rows, 0, runner.position_axes, self.widths)
        dev = runner.rt.device
        self.host = torch.zeros(lay.total, dtype=torch.int32).pin_memory()
        self.np = self.host.numpy()
        self.dev = torch.zeros(lay.total, dtype=torch.int32, device=dev)
        ar = np.arange(rows, dtype=np.int32)
        for name, value in (("row_seg", ar), ("seg_row0", ar), ("seg_rows", 1), ("logit_rows", ar), ("decode_rows", ar)):
            lay.part(self.np, name)[:] = value
        self.info = lay.info(self.dev, list(range(rows)), [1] * rows, [0] * rows, [0] * rows, span, True)
        self.info.max_context = span
        self.copied = torch.cuda.Event()
        # what the pinned block tables hold: the request of every row and how many of its pages (per group), so that
        # a step writes only what is new (`CacheManager.table_version` changes when pages were taken away)
        self.row_key: List[Optional[tuple]] = [None] * rows
        self.row_pages = [[0] * rows for _ in self.widths]
        self.rows_used = rows
        for g in range(len(self.widths)):
            lay.table(self.np, g)[:] = runner.pad_pages[g]
        self.fill([])
        self.upload()
        views = runner.bind_views(self.info)
        native = runner.native
        # one eager run on a side stream (allocations settle, the executor's work space has its size), then the capture
        side = torch.cuda.Stream(device=dev)
        side.wait_stream(torch.cuda.current_stream(dev))
        with torch.cuda.stream(side):
            runner.forward(self.info)
        torch.cuda.current_stream(dev).wait_stream(side)
        torch.cuda.synchronize(dev)
        # Two graphs: a short head (the embedding and the first layers) and the rest.  Launching a graph costs the
        # host time in proportion to its launches, and the GPU starts only when the launch call is through: with the
        # head launched first, the long launch of the rest overlaps with the head's work on the GPU.
        model = runner.model
        n_plan = len(model.spec.plan)
        cut = min(HEAD_ENTRIES, n_plan - 1) if n_plan > 1 else n_plan
        self.graphs = [torch.cuda.CUDAGraph(), torch.cuda.CUDAGraph()] if cut < n_plan else [torch.cuda.CUDAGraph()]
        # No garbage collection while the stream is capturing: a collection may free device objects of engines that
        # are no longer used (other graphs, events), which is not allowed during a capture and ends the process.
        gc_was_on = gc.isenabled()
        gc.collect()
        gc.disable()
        if native is not None:
            self.logits = torch.empty((rows, runner.vocab_size), dtype=torch.float32, device=dev)
        try:
            with torch.cuda.graph(self.graphs[0]):
                if native is not None:
                    native.begin(self.info)
                    native.run_range(0, cut)
                    if len(self.graphs) == 1:
                        native.finish(self.logits)
                else:
                    x = model.embed(self.info)
                    left = model.run_plan(x, self.info, views, 0, cut, None)
                    if len(self.graphs) == 1:
                        self.logits = model.logits(x, self.info)
            if len(self.graphs) == 2:
                with torch.cuda.graph(self.graphs[1], pool=self.graphs[0].pool()):
                    if native is not None:
                        native.run_range(cut, n_plan)
                        native.finish(self.logits)
                    else:
                        model.run_plan(x, self.info, views, cut, n_plan, left)
                        self.logits = model.logits(x, self.info)
        finally:
            if gc_was_on:
                gc.enable()
        torch.cuda.synchronize(dev)

    def _part(self, name: str) -> np.ndarray:
        return self.layout.part(self.np, name)

    def fill(self, seqs: Sequence[Hashable]) -> None:
        """Positions, state slots and block tables of the requests `seqs`, one row each (tokens: `set_tokens`)."""
        r = self.runner
        cache = r.cache
        n = len(seqs)
        self.copied.synchronize()      # the last upload has read the pinned buffer
        tokens, positions, pos0, slots = (self._part(k) for k in ("tokens", "positions", "seg_pos0", "state_slots"))
        tokens[n:] = 0
        positions[n:] = 0
        pos0[n:] = 0
        slots[n:] = cache.max_requests
        for i, seq in enumerate(seqs):
            positions[i] = pos0[i] = cache.length(seq)
            slots[i] = cache.slot_of(seq)
        if self.layout.axes > 1:     # every axis carries the token's place in its request
            self._part("position_axes").reshape(self.rows, self.layout.axes)[:] = positions[:, None]
        keys = [(seq, cache.table_version(seq)) for seq in seqs]
        used = max(n, self.rows_used)
        for g, w in enumerate(self.widths):
            bt = self.layout.table(self.np, g)
            pad = r.pad_pages[g]
            windowed = getattr(cache.paged_groups[g].need, "window", None) is not None
            if used > n:
                bt[n:used] = pad           # rows that held a request last time and hold none now
            held = self.row_pages[g]
            for i, seq in enumerate(seqs):
                t = cache.block_table(seq, g)
                k = len(t)
                row = bt[i]
                if not windowed and self.row_key[i] == keys[i] and held[i] <= k:
                    if k > held[i]:        # the same request with the same pages as last time: only the new ones
                        row[held[i]:k] = t[held[i]:]
                else:
                    row[:k] = t
                    row[k:] = pad
                    if windowed:
                        row[:k][row[:k] < 0] = pad
                held[i] = k
        self.row_key[:n] = keys
        for i in range(n, used):
            self.row_key[i] = None
        self.rows_used = n

    def set_tokens(self, tokens: Sequence[int]) -> None:
        self._part("tokens")[:len(tokens)] = tokens

    def upload(self) -> None:
        self.dev.copy_(self.host, non_blocking=True)
        self.copied.record()

    def replay(self) -> None:
        for g in self.graphs:
            g.replay()
