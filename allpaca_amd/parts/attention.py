"""Grouped-query attention over the paged cache.

Per row: q = h Wq^T, k = h Wk^T, v = h Wv^T (no bias); q and k are turned by the
position encoding before k is cached; query head j reads kv head j // (H/Hk);
score = (q.k)/sqrt(d) on the finished dot product; keys at positions <= the
row's own (of the last `window` positions if a window is set); softmax in
32-bit; out = sum p V; residual += out Wo^T
(crates/allpaca-core/src/model.rs:8528-8684, crates/allpaca-cpu/src/kernels.rs:293-356)."""
from __future__ import annotations

from typing import Dict, Mapping, Optional

import torch

from ..kernels import ops
from .base import MIXERS, POSITION_ENCODINGS, Mixer, PagedKV, Runtime, as_normed, build_part, to_device
from .spec import ParamSpec, PartSpec


@MIXERS.register("attention")
class Attention(Mixer):
    graph_safe = True
    takes_normed_input = True
    emits_next_norm = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 position: Optional[PartSpec] = None, window: Optional[int] = None, scale: Optional[float] = None):
        if num_heads % num_kv_heads:
            raise ValueError(f"attention: {num_heads} heads are not a multiple of {num_kv_heads} kv heads")
        self.D, self.H, self.Hk, self.d = int(hidden_size), int(num_heads), int(num_kv_heads), int(head_dim)
        self.window = int(window) if window else None
        self.scale = float(scale) if scale is not None else None
        self.position = build_part(POSITION_ENCODINGS, position) if position is not None else None
        self.graph_safe = self.position is None or bool(self.position.graph_safe)
        self.q_off, self.k_off, self.v_off = 0, self.H * self.d, (self.H + self.Hk) * self.d
        self.qkv_width = (self.H + 2 * self.Hk) * self.d

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {
            "q_proj.weight": ParamSpec((self.H * self.d, self.D)),
            "k_proj.weight": ParamSpec((self.Hk * self.d, self.D)),
            "v_proj.weight": ParamSpec((self.Hk * self.d, self.D)),
            "o_proj.weight": ParamSpec((self.D, self.H * self.d)),
        }

    def cache_need(self):
        return PagedKV(self.Hk, self.d, self.window)

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        self.rt = rt
        parts = [tensors["q_proj.weight"], tensors["k_proj.weight"], tensors["v_proj.weight"]]
        dt = parts[0].dtype if all(p.dtype == parts[0].dtype for p in parts) else torch.float32
        # one [(H + 2 Hk) d, D] matrix: a single product gives q, k and v of a row
        self.w_qkv = ops.prepare_matrix(torch.cat([to_device(p, rt, dt) for p in parts], dim=0), rt.dtype)
        self.w_o = ops.prepare_matrix(to_device(tensors["o_proj.weight"], rt), rt.dtype)
        if self.position is not None:
            self.position.bind({}, rt)

    def forward_add(self, h, step, cache, residual: torch.Tensor, emit=None) -> None:
        h = as_normed(h)
        T = h.shape[0]
        qkv = torch.empty((T, self.qkv_width), dtype=self.rt.dtype, device=h.device)
        fused = self.position.fused() if self.position is not None else None
        rot, table = fused if fused is not None else (0, None)
        kv = cache.kv if cache.writes else None
        # few rows, whole heads rotated, an own cache: one kernel gives q, k, v, rotates and fills the pages
        if (kv is not None and rot == self.d and h.product(
                lambda a, pre: ops.qkv_rope_write(a, pre, self.w_qkv, qkv, self.H, self.Hk, self.d, table,
                                                  step.positions, step.row_seg, cache.block_table, kv,
                                                  cache.page_tokens))):
            pass
        else:
            h.linear(self.w_qkv, qkv)
            if self.position is not None and fused is None:
                self.position.apply(qkv, self.q_off, self.k_off, self.H, self.Hk, self.d,
                                    step.positions if step.position_axes is None else step.position_axes)
            if kv is not None or rot:
                ops.rope_kv_write(qkv, self.q_off, self.k_off, self.v_off, self.H, self.Hk, self.d, rot, table,
                                  step.positions, step.row_seg, cache.block_table, kv, cache.page_tokens)
        attn = torch.empty((T, self.H * self.d), dtype=self.rt.dtype, device=h.device)
        ops.paged_attention(qkv, self.q_off, attn, self.H, self.Hk, self.d, cache.kv, cache.page_tokens,
                            cache.block_table, step, window=self.window or 0, scale=self.scale)
        ops.linear(attn, self.w_o, residual, accumulate=True, emit=emit)

    def native_desc(self):
        if type(self) is not Attention:
            return None
        fused = self.position.fused() if self.position is not None else (0, None)
        if fused is None:           # an encoding that transforms q and k itself: walked in Python
            return None
        rot, table = fused
        return {"kind": "attention", "w_qkv": self.w_qkv, "w_o": self.w_o, "H": self.H, "Hk": self.Hk, "d": self.d,
                "window": self.window or 0, "scale": self.scale or 0.0, "rot": int(rot), "cos_sin": table}

    def forward(self, h, step, cache):
        out = torch.zeros((h.shape[0], self.D), dtype=torch.float32, device=h.device)
        self.forward_add(h, step, cache, out)
        return out
