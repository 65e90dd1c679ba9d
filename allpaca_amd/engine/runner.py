"""The step function: a batch of (request, its next tokens) in, logits at the
wanted places out.  It runs only the tokens it is given, as one batch, against
the cache that earlier steps left; portions of prompts stand beside single
decoded tokens, cut anywhere.

The reference has three forwards (one token, one sequence's rows, many
sequences' rows: crates/allpaca-core/src/model.rs:8195, 8894, 8839) and never
mixes a prompt portion with decode rows in one of them
(crates/allpaca-core/src/engine.rs:5451-5607); this is the one generalisation."""
from __future__ import annotations

from typing import Dict, Hashable, List, Optional, Sequence

import torch

from ..cache import CacheManager, CacheStorage, OutOfPages, PagedView, StateView
from ..models.decoder import DecoderModel
from .batch import Entry, StepInfo, pack_step


class StepError(ValueError):
    pass


class ModelRunner:
    def __init__(self, model: DecoderModel, page_tokens: int, num_pages, max_requests: int,
                 kv_dtype: Optional[torch.dtype] = None):
        if model.rt is None:
            raise StepError("the model has no weights bound")
        self.model = model
        self.rt = model.rt
        self.cache = CacheManager(model.cache_needs(), page_tokens, num_pages, max_requests)
        self.storage = CacheStorage(self.cache, kv_dtype or self.rt.dtype, self.rt.device)
        self.views = self.storage.views(model.spec.plan)
        self.pad_pages = [self.storage.dummy_page(g) for g in range(len(self.cache.paged_groups))]
        self.vocab_size = model.spec.vocab_size
        self.steps = 0

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

    def step(self, entries: Sequence[Entry]) -> Optional[torch.Tensor]:
        """Runs one batch; returns float32 logits [sum of wanted places, vocab] (device), or None."""
        if not entries:
            return None
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
        info = self.pack(entries)
        logits = self.model.forward(info, self.bind_views(info))
        for e in entries:
            self.cache.commit(e.seq, len(e.tokens))
        self.steps += 1
        return logits

    def pack(self, entries: Sequence[Entry]) -> StepInfo:
        pos0 = [self.cache.length(e.seq) for e in entries]
        slots = [self.cache.slot_of(e.seq) for e in entries]
        tables = [[self.cache.block_table(e.seq, g) for e in entries] for g in range(len(self.cache.paged_groups))]
        return pack_step(entries, pos0, slots, tables, self.rt.device, self.pad_pages)

    def bind_views(self, info: StepInfo) -> list:
        for v in self.views:
            if isinstance(v, PagedView):
                v.block_table = info.block_tables[v.group]
            elif isinstance(v, StateView):
                v.slots = info.state_slots
                v.slots_host = info.host_slots
        return self.views
