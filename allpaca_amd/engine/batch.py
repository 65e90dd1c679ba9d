"""One step's batch: for each request its next tokens and the places among them
whose logits are wanted; and the same on the device, as the kernels read it.

The reference describes a batch as `tokens` plus `SeqRows{start_pos, n_rows,
page_ids}` per sequence (crates/allpaca-core/src/model.rs:36-42, 10865-10885);
here every row also carries its own position and segment, so rotation, cache
write and attention take one launch for the whole mixed batch.

The description lives in one int32 buffer on the device.  `StepLayout` says
which piece of the buffer is which array, and `StepLayout.info` is the only
place where a `StepInfo` is made from such a buffer: the packer of ordinary
steps and the replayed decode graphs both go through it, so an array added here
reaches both."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

import numpy as np
import torch


@dataclass
class Entry:
    """A request's part of a step."""
    seq: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()          # indices into `tokens` whose logits are returned, in this order
    # For models whose position encoding takes more than one axis: [len(tokens)][axes] positions of the tokens on
    # those axes.  None: every axis carries the token's place in its request.
    positions: Optional[Sequence[Sequence[int]]] = None


@dataclass
class StepInfo:
    """The batch on the device.  Rows of a segment are consecutive positions of one request."""
    n_rows: int
    n_segs: int
    tokens: torch.Tensor              # int32 [T]
    positions: torch.Tensor           # int32 [T]   place of the row in its request (where its keys and values go)
    row_seg: torch.Tensor             # int32 [T]   segment of the row
    seg_row0: torch.Tensor            # int32 [S]   first row of the segment
    seg_rows: torch.Tensor            # int32 [S]   rows in the segment
    seg_pos0: torch.Tensor            # int32 [S]   position of the segment's first row
    state_slots: torch.Tensor         # int32 [S]
    logit_rows: Optional[torch.Tensor]  # int32 [R]
    n_logit_rows: int
    block_tables: List[torch.Tensor]  # per paged group: int32 [S, blocks]
    # int32 [T, axes] for a model whose spec names more than one position axis, else None
    position_axes: Optional[torch.Tensor] = None
    # host copies, for parts that plan on the host (and for tests)
    host_row0: List[int] = field(default_factory=list)
    host_rows: List[int] = field(default_factory=list)
    host_pos0: List[int] = field(default_factory=list)
    host_slots: List[int] = field(default_factory=list)
    max_context: int = 0              # largest (pos0 + rows) of the step
    max_rows: int = 0                 # largest segment
    decode_only: bool = False         # every segment is a single row
    # how attention kernels divide the rows: single-row segments ("decode rows") and, for longer
    # segments, tiles of at most `tile_rows` consecutive rows of one segment (the attention kernel's size)
    decode_rows: Optional[torch.Tensor] = None   # int32 [n_decode_rows] row indices; None when every row is one
    n_decode_rows: int = 0
    max_decode_context: int = 0       # largest (position + 1) among the decode rows
    tile_row0: Optional[torch.Tensor] = None     # int32 [n_tiles]
    tile_rows: Optional[torch.Tensor] = None     # int32 [n_tiles]
    n_tiles: int = 0


# the arrays of the buffer, in order; block tables follow, one per paged group
ARRAYS = ("tokens", "positions", "row_seg", "seg_row0", "seg_rows", "seg_pos0", "state_slots", "logit_rows",
          "decode_rows", "tile_row0", "tile_rows", "position_axes")


class StepLayout:
    """Where the arrays of a step lie in its int32 buffer: T rows, S segments, R wanted rows, `n_decode` single-row
    segments, `n_tiles` attention tiles, `axes` position axes (1: no array for them), block tables of the given
    widths."""

    def __init__(self, T: int, S: int, R: int, n_decode: int, n_tiles: int, axes: int, widths: Sequence[int]):
        self.T, self.S, self.R, self.n_decode, self.n_tiles, self.axes = T, S, R, n_decode, n_tiles, axes
        self.widths = list(widths)
        sizes = {"tokens": T, "positions": T, "row_seg": T, "seg_row0": S, "seg_rows": S, "seg_pos0": S,
                 "state_slots": S, "logit_rows": R, "decode_rows": n_decode, "tile_row0": n_tiles,
                 "tile_rows": n_tiles, "position_axes": T * axes if axes > 1 else 0}
        self.span: Dict[str, Tuple[int, int]] = {}
        at = 0
        for name in ARRAYS:
            self.span[name] = (at, at + sizes[name])
            at += sizes[name]
        self.table_span: List[Tuple[int, int]] = []
        for w in self.widths:
            self.table_span.append((at, at + S * w))
            at += S * w
        self.total = at

    def part(self, buffer, name: str):
        """The piece of `buffer` (a flat torch tensor or numpy array of `total` int32) that holds array `name`."""
        lo, hi = self.span[name]
        return buffer[lo:hi]

    def table(self, buffer, group: int):
        lo, hi = self.table_span[group]
        return buffer[lo:hi].reshape(self.S, self.widths[group])

    def info(self, dev: torch.Tensor, host_row0, host_rows, host_pos0, host_slots, max_decode_context: int,
             all_rows_decode: bool) -> StepInfo:
        """The `StepInfo` over the device buffer `dev` laid out like this."""
        v = {name: self.part(dev, name) for name in ARRAYS}
        return StepInfo(
            n_rows=self.T, n_segs=self.S, tokens=v["tokens"], positions=v["positions"], row_seg=v["row_seg"],
            seg_row0=v["seg_row0"], seg_rows=v["seg_rows"], seg_pos0=v["seg_pos0"], state_slots=v["state_slots"],
            logit_rows=v["logit_rows"] if self.R else None, n_logit_rows=self.R,
            block_tables=[self.table(dev, g) for g in range(len(self.widths))],
            position_axes=v["position_axes"].view(self.T, self.axes) if self.axes > 1 else None,
            decode_rows=None if all_rows_decode else v["decode_rows"], n_decode_rows=self.n_decode,
            max_decode_context=max_decode_context, tile_row0=v["tile_row0"], tile_rows=v["tile_rows"],
            n_tiles=self.n_tiles, host_row0=list(host_row0), host_rows=list(host_rows), host_pos0=list(host_pos0),
            host_slots=list(host_slots),
            max_context=max([p + n for p, n in zip(host_pos0, host_rows)] or [0]), max_rows=max(list(host_rows) or [0]),
            decode_only=all(n == 1 for n in host_rows))


def pack_step(entries: Sequence[Entry], pos0: Sequence[int], slots: Sequence[int],
              tables: Sequence[Sequence[Sequence[int]]], device: torch.device, pad_page: Sequence[int],
              min_blocks: int = 1, tile_rows: int = 64, position_axes: int = 1) -> StepInfo:
    """Builds the device-side description with one host-to-device copy.
    `tables[g][s]` is segment s's block table in paged group g; entries marked
    freed (< 0) are replaced by the group's spare page, which no live request holds.
    `tile_rows`: rows of a tile of the attention kernel that takes segments of several rows (the kernels' wrapper
    says how many); `position_axes`: axes of the model's position encoding."""
    S = len(entries)
    rows = [len(e.tokens) for e in entries]
    T = sum(rows)
    row0 = np.concatenate([[0], np.cumsum(rows)[:-1]]).astype(np.int32) if S else np.zeros(0, np.int32)
    want = np.asarray([r0 + w for e, r0 in zip(entries, row0) for w in e.want], dtype=np.int32)
    decode_rows = np.asarray([r0 for r0, n in zip(row0, rows) if n == 1], dtype=np.int32)
    t_row0, t_rows = [], []
    for r0, n in zip(row0, rows):
        if n > 1:
            for a in range(0, n, tile_rows):
                t_row0.append(r0 + a)
                t_rows.append(min(tile_rows, n - a))
    widths = [max([min_blocks] + [len(t) for t in per_seg]) for per_seg in tables]
    lay = StepLayout(T, S, int(want.size), int(decode_rows.size), len(t_row0), position_axes, widths)
    flat = np.zeros(lay.total, np.int32)
    if S:
        lay.part(flat, "tokens")[:] = np.concatenate([np.asarray(e.tokens, dtype=np.int32) for e in entries])
        positions = np.concatenate([np.arange(p, p + n, dtype=np.int32) for p, n in zip(pos0, rows)])
        lay.part(flat, "positions")[:] = positions
        lay.part(flat, "row_seg")[:] = np.repeat(np.arange(S, dtype=np.int32), rows)
        lay.part(flat, "seg_row0")[:] = row0
        lay.part(flat, "seg_rows")[:] = rows
        lay.part(flat, "seg_pos0")[:] = pos0
        lay.part(flat, "state_slots")[:] = slots
        lay.part(flat, "logit_rows")[:] = want
        lay.part(flat, "decode_rows")[:] = decode_rows
        lay.part(flat, "tile_row0")[:] = t_row0
        lay.part(flat, "tile_rows")[:] = t_rows
        if position_axes > 1:
            ax = lay.part(flat, "position_axes").reshape(T, position_axes)
            for e, r0, n in zip(entries, row0, rows):
                if e.positions is None:
                    ax[r0:r0 + n] = positions[r0:r0 + n, None]
                else:
                    given = np.asarray(e.positions, dtype=np.int32)
                    if given.shape != (n, position_axes):
                        raise ValueError(f"request {e.seq!r}: positions must be [{n}][{position_axes}], got "
                                         f"{given.shape}")
                    ax[r0:r0 + n] = given
    for g, per_seg in enumerate(tables):
        bt = lay.table(flat, g)
        bt[:] = pad_page[g]
        for s, t in enumerate(per_seg):
            if len(t):
                a = np.asarray(t, dtype=np.int32)
                bt[s, : len(t)] = np.where(a < 0, pad_page[g], a)
    host = torch.from_numpy(flat).pin_memory() if device.type == "cuda" else torch.from_numpy(flat)
    dev = host.to(device, non_blocking=False)
    return lay.info(dev, row0.tolist(), rows, list(pos0), list(slots),
                    max([p + 1 for p, n in zip(pos0, rows) if n == 1] or [0]), int(decode_rows.size) == T)
