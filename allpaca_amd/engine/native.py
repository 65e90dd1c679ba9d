"""A model's steps on the compiled plan executor (`csrc/host/exec.cpp`).

`NativeProgram.of(model, views)` asks every part of the model to describe itself (`Part.native_desc`) and, if all
do, builds the executor's program: layers, plan entries with their pages, embedding, final norm, head.  A step is
then one call, `forward(info)`, which issues every launch from C++ over a work space that is sized by a run
without launches (`apc_host_step_bytes`) and grows only when a step needs more than any before it.  Logits come
back in a tensor of the caller's; everything between lives in the work space."""
from __future__ import annotations

import ctypes
from typing import List, Optional

import torch

from ..cache import PagedView
from ..kernels import host as H
from ..kernels import ops, tuned
from ..kernels.packing import PackedWeight

_CODES = {torch.float32: 0, torch.bfloat16: 1, torch.int32: 2}


def _matrix(w, keep: list) -> H.ApcMatrix:
    if isinstance(w, PackedWeight):
        keep.append(w.data)
        return H.ApcMatrix(w.data.data_ptr(), 1, 1, w.N, w.K, w.chunks, 0)
    if not (isinstance(w, torch.Tensor) and w.dim() == 2 and w.is_cuda and w.stride(1) == 1 and w.dtype in _CODES):
        raise TypeError("a weight matrix must be a tiled matrix or a row-major tensor on the GPU")
    keep.append(w)
    return H.ApcMatrix(w.data_ptr(), 0, _CODES[w.dtype], w.shape[0], w.shape[1], 0, w.stride(0))


class NativeProgram:
    def __init__(self):
        raise TypeError("use NativeProgram.of")

    @classmethod
    def of(cls, model, views) -> Optional["NativeProgram"]:
        """The program of `model` over the cache views of its plan entries, or None if some part is not one the
        executor knows (or some plan entry has no pages of keys and values)."""
        spec, rt = model.spec, model.rt
        if rt is None or rt.device.type != "cuda" or rt.dtype not in (torch.float32, torch.bfloat16):
            return None
        emb, fin, head = model.embedding.native_desc(), model.final_norm.native_desc(), model.head.native_desc()
        blocks = [b.native_desc() for b in model.blocks]
        if (emb is None or fin is None or head is None or any(b is None for b in blocks)
                or emb["kind"] != "token_table" or fin["kind"] != "rmsnorm" or head["kind"] != "linear"
                or getattr(spec, "position_axes", 1) != 1):
            return None
        if any(not isinstance(v, PagedView) or v.kv.dim() != 5 or not v.kv.is_contiguous() or v.group >= 8
               or v.kv.dtype not in _CODES for v in views):
            return None
        self = object.__new__(cls)
        self.lib = L = H.load()
        self.keep: list = []            # every tensor the program points into
        self.device = rt.device
        self.run_dtype = rt.dtype
        self.vocab = spec.vocab_size
        self.hidden = spec.hidden_size
        self.n_plan = len(spec.plan)
        e_m, h_m = _matrix(emb["weight"], self.keep), _matrix(head["weight"], self.keep)
        if e_m.K != self.hidden or h_m.K != self.hidden or h_m.N != self.vocab:
            return None
        self.keep.append(fin["weight"])
        self.handle = L.apc_host_program_new(self.hidden, self.vocab, _CODES[rt.dtype], ctypes.byref(e_m),
                                             fin["weight"].data_ptr(), float(fin["eps"]), ctypes.byref(h_m))
        if not self.handle:
            return None
        for b, d in zip(model.blocks, blocks):
            a, f = d["mixer"], d["ffn"]
            layer = H.ApcLayer()
            layer.norm1_w, layer.norm1_eps = d["mixer_norm"]["weight"].data_ptr(), float(d["mixer_norm"]["eps"])
            layer.norm2_w, layer.norm2_eps = d["ffn_norm"]["weight"].data_ptr(), float(d["ffn_norm"]["eps"])
            self.keep += [d["mixer_norm"]["weight"], d["ffn_norm"]["weight"]]
            layer.w_qkv, layer.w_o = _matrix(a["w_qkv"], self.keep), _matrix(a["w_o"], self.keep)
            layer.H, layer.Hk, layer.d, layer.window = a["H"], a["Hk"], a["d"], int(a["window"])
            layer.scale, layer.rot = float(a["scale"]), int(a["rot"])
            if a["rot"]:
                table = a["cos_sin"]
                if not (table.dtype == torch.float32 and table.is_contiguous()
                        and tuple(table.shape[1:]) == (2, a["rot"] // 2)):
                    return self._give_up()
                self.keep.append(table)
                layer.cos_sin = table.data_ptr()
            gu = f["w_gate_up"]
            if isinstance(gu, tuple):
                layer.w_gate, layer.w_up = _matrix(gu[0], self.keep), _matrix(gu[1], self.keep)
            else:
                layer.w_gate = _matrix(gu, self.keep)
            layer.w_down, layer.F = _matrix(f["w_down"], self.keep), int(f["F"])
            if L.apc_host_program_add_layer(self.handle, ctypes.byref(layer)) < 0:
                return self._give_up()
        for e, v in zip(spec.plan, views):
            a = blocks[e.block]["mixer"]
            if tuple(v.kv.shape[1:]) != (2, a["Hk"], v.page_tokens, a["d"]) or (v.window or 0) != a["window"]:
                return self._give_up()
            self.keep.append(v.kv)
            entry = H.ApcPlanEntry(e.block, v.kv.data_ptr(), _CODES[v.kv.dtype], v.group, v.page_tokens,
                                   1 if v.writes else 0)
            if L.apc_host_program_add_entry(self.handle, ctypes.byref(entry)) < 0:
                return self._give_up()
        self.counters = tuned._pair_counters(self.device, 4096)
        self.counters.zero_()      # a count that a failed launch left would hold up every later step
        self._set_tunables()
        self.arenas: List[torch.Tensor] = []
        self.arena: Optional[torch.Tensor] = None
        self._step = H.ApcStep()
        self.launches = 0
        return self

    def _give_up(self):
        self.close()
        return None

    def close(self) -> None:
        if getattr(self, "handle", None):
            self.lib.apc_host_program_free(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @staticmethod
    def _rules() -> tuple:
        """The numbers the kernels' wrappers keep as module constants (tests and measurements move them)."""
        return (tuned.WHOLE_MIN_PAIRS, tuned.LAST_BLOCK_MERGES, tuned.WIDE_TILES, tuned.KEY_SPLITS_MAX,
                tuned.KEY_RANGE_MIN, ops.FORCE_PLAIN)

    def _set_tunables(self) -> None:
        t = H.ApcTunables(int(min(tuned.WHOLE_MIN_PAIRS, 1 << 30)), int(bool(tuned.LAST_BLOCK_MERGES)),
                          int(bool(tuned.WIDE_TILES)), int(tuned.KEY_SPLITS_MAX), int(tuned.KEY_RANGE_MIN),
                          int(bool(ops.FORCE_PLAIN)))
        self._tunables = self._rules()
        self.lib.apc_host_program_tunables(self.handle, ctypes.byref(t), self.counters.data_ptr(),
                                           self.counters.numel())

    # ---- a step ------------------------------------------------------------------------------------------------
    def describe(self, info, into: Optional[H.ApcStep] = None) -> H.ApcStep:
        s = into if into is not None else H.ApcStep()
        s.T, s.S, s.R, s.n_decode, s.n_tiles = info.n_rows, info.n_segs, info.n_logit_rows, info.n_decode_rows, info.n_tiles
        for name in H.STEP_ARRAYS:
            t = getattr(info, name)
            setattr(s, name, t.data_ptr() if t is not None and t.numel() else None)
        s.n_groups = len(info.block_tables)
        for g, bt in enumerate(info.block_tables):
            s.table[g] = bt.data_ptr()
            s.table_width[g] = bt.shape[1]
        s.max_decode_context = info.max_decode_context
        s.all_rows_decode = 1 if info.decode_rows is None else 0
        s.max_prompt_keys = max([p + n for p, n in zip(info.host_pos0, info.host_rows) if n > 1] or [0])
        return s

    def room_for(self, s: H.ApcStep) -> torch.Tensor:
        """The work space, grown if this step needs more than any before (the old one stays while graphs point into it)."""
        need = self.lib.apc_host_step_bytes(self.handle, ctypes.byref(s))
        if need < 0:
            H.check(int(need), "sizing a step")
        if self.arena is None or self.arena.numel() < need:
            self.arena = torch.empty(int(need * 1.25) + 4096, dtype=torch.uint8, device=self.device)
            self.arenas.append(self.arena)
        return self.arena

    def reserve(self, rows: int, info_like) -> None:
        """Sizes the work space for a step like `info_like` once, before serving starts."""
        self.room_for(self.describe(info_like))

    def forward(self, info) -> Optional[torch.Tensor]:
        """The whole step: float32 logits [wanted rows, vocab] or None."""
        if self._rules() != self._tunables:
            self._set_tunables()
        s = self.describe(info, self._step)
        arena = self.room_for(s)
        logits = (torch.empty((s.R, self.vocab), dtype=torch.float32, device=self.device) if s.R else None)
        H.check(self.lib.apc_host_step(self.handle, ctypes.byref(s), arena.data_ptr(), arena.numel(),
                                       logits.data_ptr() if logits is not None else None, ops._stream()), "a step")
        return logits

    # the same in pieces, for a caller that records a step into more than one graph
    def begin(self, info) -> None:
        s = self.describe(info)
        arena = self.room_for(s)
        self._piece = (s, arena)      # both must live until the last piece has been issued
        H.check(self.lib.apc_host_step_begin(self.handle, ctypes.byref(s), arena.data_ptr(), arena.numel(),
                                             ops._stream()), "a step's embedding")

    def run_range(self, lo: int, hi: int) -> None:
        H.check(self.lib.apc_host_step_range(self.handle, lo, hi), "a range of the plan")

    def finish(self, logits: Optional[torch.Tensor]) -> None:
        H.check(self.lib.apc_host_step_finish(self.handle, logits.data_ptr() if logits is not None else None),
                "the head")

    # ---- per-launch timers -------------------------------------------------------------------------------------
    def timing(self, on: bool) -> None:
        self.lib.apc_host_timing(self.handle, 1 if on else 0)

    def timing_report(self) -> List[tuple]:
        """[(launch, microseconds)] in launch order, for the steps run since `timing(True)`; waits for the GPU."""
        text = self.lib.apc_host_timing_report(self.handle).decode()
        return [(name, float(us)) for name, us in (line.split("\t") for line in text.splitlines() if line)]
