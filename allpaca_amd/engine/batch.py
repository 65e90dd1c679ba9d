"""One step's batch: for each request its next tokens and the places among them
whose logits are wanted; and the same on the device, as the kernels read it.

The reference describes a batch as `tokens` plus `SeqRows{start_pos, n_rows,
page_ids}` per sequence (crates/allpaca-core/src/model.rs:36-42, 10865-10885);
here every row also carries its own position and segment, so rotation, cache
write and attention take one launch for the whole mixed batch."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence

import numpy as np
import torch


@dataclass
class Entry:
    """A request's part of a step."""
    seq: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()          # indices into `tokens` whose logits are returned, in this order


@dataclass
class StepInfo:
    """The batch on the device.  Rows of a segment are consecutive positions of one request."""
    n_rows: int
    n_segs: int
    tokens: torch.Tensor              # int32 [T]
    positions: torch.Tensor           # int32 [T]   position of the row in its request
    row_seg: torch.Tensor             # int32 [T]   segment of the row
    seg_row0: torch.Tensor            # int32 [S]   first row of the segment
    seg_rows: torch.Tensor            # int32 [S]   rows in the segment
    seg_pos0: torch.Tensor            # int32 [S]   position of the segment's first row
    state_slots: torch.Tensor         # int32 [S]
    logit_rows: Optional[torch.Tensor]  # int32 [R]
    n_logit_rows: int
    block_tables: List[torch.Tensor]  # per paged group: int32 [S, blocks]
    # host copies, for parts that plan on the host (and for tests)
    host_row0: List[int] = field(default_factory=list)
    host_rows: List[int] = field(default_factory=list)
    host_pos0: List[int] = field(default_factory=list)
    host_slots: List[int] = field(default_factory=list)
    max_context: int = 0              # largest (pos0 + rows) of the step
    max_rows: int = 0                 # largest segment
    decode_only: bool = False         # every segment is a single row
    # how attention kernels divide the rows: single-row segments ("decode rows") and, for longer
    # segments, tiles of at most TILE_ROWS consecutive rows of one segment
    decode_rows: Optional[torch.Tensor] = None   # int32 [n_decode_rows] row indices; None when every row is one
    n_decode_rows: int = 0
    max_decode_context: int = 0       # largest (position + 1) among the decode rows
    tile_row0: Optional[torch.Tensor] = None     # int32 [n_tiles]
    tile_rows: Optional[torch.Tensor] = None     # int32 [n_tiles]
    n_tiles: int = 0


TILE_ROWS = 64    # rows of an attention tile (must match the prefill kernel's)


def pack_step(entries: Sequence[Entry], pos0: Sequence[int], slots: Sequence[int],
              tables: Sequence[Sequence[Sequence[int]]], device: torch.device, pad_page: Sequence[int],
              min_blocks: int = 1) -> StepInfo:
    """Builds the device-side description with one host-to-device copy.
    `tables[g][s]` is segment s's block table in paged group g; entries marked
    freed (< 0) are replaced by the group's spare page, which no live request holds."""
    S = len(entries)
    rows = [len(e.tokens) for e in entries]
    T = sum(rows)
    row0 = np.concatenate([[0], np.cumsum(rows)[:-1]]).astype(np.int32) if S else np.zeros(0, np.int32)
    tokens = np.concatenate([np.asarray(e.tokens, dtype=np.int32) for e in entries]) if S else np.zeros(0, np.int32)
    positions = np.concatenate([np.arange(p, p + n, dtype=np.int32) for p, n in zip(pos0, rows)])
    row_seg = np.repeat(np.arange(S, dtype=np.int32), rows)
    logit_rows = np.asarray([r0 + w for e, r0 in zip(entries, row0) for w in e.want], dtype=np.int32)
    blocks = []
    for g, per_seg in enumerate(tables):
        width = max([min_blocks] + [len(t) for t in per_seg])
        bt = np.full((S, width), pad_page[g], dtype=np.int32)
        for s, t in enumerate(per_seg):
            if len(t):
                a = np.asarray(t, dtype=np.int32)
                bt[s, : len(t)] = np.where(a < 0, pad_page[g], a)
        blocks.append(bt)
    decode_rows = np.asarray([r0 for r0, n in zip(row0, rows) if n == 1], dtype=np.int32)
    t_row0, t_rows = [], []
    for r0, n in zip(row0, rows):
        if n > 1:
            for a in range(0, n, TILE_ROWS):
                t_row0.append(r0 + a)
                t_rows.append(min(TILE_ROWS, n - a))
    parts = [tokens, positions, row_seg, row0, np.asarray(rows, np.int32), np.asarray(pos0, np.int32),
             np.asarray(slots, np.int32), logit_rows, decode_rows, np.asarray(t_row0, np.int32),
             np.asarray(t_rows, np.int32)] + [b.reshape(-1) for b in blocks]
    flat = np.concatenate(parts) if parts else np.zeros(0, np.int32)
    host = torch.from_numpy(flat).pin_memory() if device.type == "cuda" else torch.from_numpy(flat)
    dev = host.to(device, non_blocking=False)
    cuts = np.cumsum([0] + [p.size for p in parts])
    v = [dev[cuts[i]: cuts[i + 1]] for i in range(len(parts))]
    return StepInfo(
        n_rows=T, n_segs=S, tokens=v[0], positions=v[1], row_seg=v[2], seg_row0=v[3], seg_rows=v[4], seg_pos0=v[5],
        state_slots=v[6], logit_rows=v[7] if logit_rows.size else None, n_logit_rows=int(logit_rows.size),
        block_tables=[v[11 + g].view(S, blocks[g].shape[1]) for g in range(len(blocks))],
        decode_rows=None if decode_rows.size == T else v[8], n_decode_rows=int(decode_rows.size),
        max_decode_context=max([p + 1 for p, n in zip(pos0, rows) if n == 1] or [0]),
        tile_row0=v[9], tile_rows=v[10], n_tiles=len(t_row0),
        host_row0=row0.tolist(), host_rows=list(rows), host_pos0=list(pos0), host_slots=list(slots),
        max_context=max([p + n for p, n in zip(pos0, rows)] or [0]), max_rows=max(rows or [0]),
        decode_only=all(n == 1 for n in rows))
