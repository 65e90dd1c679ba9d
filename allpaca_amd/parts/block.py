"""Arrangements: how the parts of one layer are wired on the residual stream.
The residual stream x is float32 [T, D]; parts read a normalised copy in the
run's element type and add their output into x in 32-bit."""
from __future__ import annotations

from typing import Dict, Mapping

import torch

from .base import ARRANGEMENTS, FEED_FORWARDS, MIXERS, NORMS, Part, build_part
from .spec import BlockSpec


class Block:
    """The built parts of one layer and the function that runs them."""

    def __init__(self, spec: BlockSpec):
        self.spec = spec
        arrangement = ARRANGEMENTS.get(spec.arrangement)
        self.parts: Dict[str, Part] = {}
        for role, pspec in spec.parts.items():
            self.parts[role] = build_part(arrangement.registries[role], pspec)
        self.run = lambda x, step, cache: arrangement.run(self.parts, x, step, cache)

    @property
    def mixer(self):
        return self.parts["mixer"]

    def param_specs(self):
        out = {}
        for role, part in self.parts.items():
            prefix = self.spec.weight_prefix + self.spec.parts[role].weight_prefix
            for name, ps in part.param_specs().items():
                out[prefix + name] = ps
        return out

    def bind(self, tensors: Mapping[str, torch.Tensor], rt) -> None:
        for role, part in self.parts.items():
            prefix = self.spec.weight_prefix + self.spec.parts[role].weight_prefix
            local = {name: tensors[prefix + name] for name in part.param_specs() if prefix + name in tensors}
            part.bind(local, rt)


@ARRANGEMENTS.register("pre_norm")
class PreNorm:
    """x += mixer(norm(x)); x += ffn(norm(x))  (crates/allpaca-core/src/model.rs:8447-8455, 8667-8696)."""
    registries = {"mixer_norm": NORMS, "mixer": MIXERS, "ffn_norm": NORMS, "ffn": FEED_FORWARDS}

    @staticmethod
    def run(parts, x: torch.Tensor, step, cache) -> None:
        rt = parts["mixer"].rt
        h = torch.empty(x.shape, dtype=rt.dtype, device=x.device)
        parts["mixer_norm"].forward(x, h)
        parts["mixer"].forward_add(h, step, cache, x)
        parts["ffn_norm"].forward(x, h)
        parts["ffn"].forward_add(h, step, x)
