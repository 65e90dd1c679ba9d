"""SwiGLU feed-forward: a = silu(h Wg^T) * (h Wu^T), residual += a Wd^T, no bias,
silu(z) = z / (1 + exp(-z)) (crates/allpaca-core/src/model.rs:5664-5705,
crates/allpaca-cpu/src/kernels.rs:869-871)."""
from __future__ import annotations

from typing import Dict, Mapping

import torch

from ..kernels import ops
from .base import FEED_FORWARDS, FeedForward, Runtime, as_normed, to_device
from .spec import ParamSpec


@FEED_FORWARDS.register("swiglu")
class SwiGLU(FeedForward):
    graph_safe = True

    takes_normed_input = True
    emits_next_norm = True

    def __init__(self, hidden_size: int, intermediate_size: int):
        self.D, self.F = int(hidden_size), int(intermediate_size)

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {
            "gate_proj.weight": ParamSpec((self.F, self.D)),
            "up_proj.weight": ParamSpec((self.F, self.D)),
            "down_proj.weight": ParamSpec((self.D, self.F)),
        }

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        self.rt = rt
        g, u = tensors["gate_proj.weight"], tensors["up_proj.weight"]
        dt = g.dtype if g.dtype == u.dtype else torch.float32
        # one pass over h gives both branches: the pair of tiled matrices for the MFMA kernels, else
        # [2F, D] (gate rows, then up rows)
        wg, wu = ops.prepare_matrix(to_device(g, rt, dt), rt.dtype), ops.prepare_matrix(to_device(u, rt, dt), rt.dtype)
        if isinstance(wg, torch.Tensor):
            self.w_gate_up = torch.cat([wg, wu], dim=0).contiguous()
        else:
            self.w_gate_up = (wg, wu)
        self.w_down = ops.prepare_matrix(to_device(tensors["down_proj.weight"], rt), rt.dtype)

    def forward_add(self, h, step, residual: torch.Tensor, emit=None) -> None:
        h = as_normed(h)
        act = torch.empty((h.shape[0], self.F), dtype=self.rt.dtype, device=h.device)
        h.swiglu(self.w_gate_up, act)
        ops.linear(act, self.w_down, residual, accumulate=True, emit=emit)

    def native_desc(self):
        if type(self) is not SwiGLU:
            return None
        return {"kind": "swiglu", "w_gate_up": self.w_gate_up, "w_down": self.w_down, "F": self.F}

    def forward(self, h, step):
        out = torch.zeros((h.shape[0], self.D), dtype=torch.float32, device=h.device)
        self.forward_add(h, step, out)
        return out
