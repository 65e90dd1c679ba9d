"""Arrangements: how the parts of one layer are wired on the residual stream.
The residual stream x is float32 [T, D]; parts read a normalised copy in the
run's element type and add their output into x in 32-bit."""
from __future__ import annotations

from typing import Dict, Mapping

import torch

from .base import ARRANGEMENTS, FEED_FORWARDS, MIXERS, NORMS, NormEmit, NormedInput, Part, build_part
from .spec import BlockSpec


class Block:
    """The built parts of one layer and the function that runs them."""

    def __init__(self, spec: BlockSpec):
        self.spec = spec
        arrangement = ARRANGEMENTS.get(spec.arrangement)
        self.parts: Dict[str, Part] = {}
        for role, pspec in spec.parts.items():
            self.parts[role] = build_part(arrangement.registries[role], pspec)
        self.arrangement = arrangement
        self.chains_norms = bool(getattr(arrangement, "chains_norms", False))

    def run(self, x: torch.Tensor, step, cache, pre=None, next_norm=None):
        """Runs the layer on the residual stream x.  `pre`: what the layer before left for this layer's first norm
        (a filled `NormEmit`) or None; `next_norm`: the norm that reads x after this layer.  Returns what this
        layer left for `next_norm`, or None.  Only arrangements with `chains_norms` take part in that."""
        if self.chains_norms:
            return self.arrangement.run(self.parts, x, step, cache, pre=pre, next_norm=next_norm)
        self.arrangement.run(self.parts, x, step, cache)
        return None

    def first_norm(self):
        """The norm that reads the residual stream first in this layer, if the layer can use what the product
        before it leaves for that norm."""
        return self.arrangement.first_norm(self.parts) if self.chains_norms else None

    @property
    def mixer(self):
        return self.parts["mixer"]

    def cache_needs(self) -> Dict[str, object]:
        """role -> what that part needs of the cache manager, for every part of the layer that keeps something per
        request (`cache_need()` answering other than None): attention heads beside recurrent heads are two roles with
        a need each."""
        out = {}
        for role, part in self.parts.items():
            ask = getattr(part, "cache_need", None)
            need = ask() if callable(ask) else None
            if need is not None:
                out[role] = need
        return out

    def native_desc(self):
        describe = getattr(self.arrangement, "native_desc", None)
        return describe(self.parts) if describe is not None else None

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
    chains_norms = True

    @staticmethod
    def first_norm(parts):
        return parts["mixer_norm"] if parts["mixer"].takes_normed_input else None

    @staticmethod
    def native_desc(parts):
        """The layer for the compiled executor, if it knows all four parts: a dict role -> the part's own description."""
        out = {role: parts[role].native_desc() for role in ("mixer_norm", "mixer", "ffn_norm", "ffn")}
        kinds = {"mixer_norm": "rmsnorm", "mixer": "attention", "ffn_norm": "rmsnorm", "ffn": "swiglu"}
        if any(d is None or d.get("kind") != kinds[role] for role, d in out.items()):
            return None
        return {"kind": "pre_norm", **out}

    @staticmethod
    def run(parts, x: torch.Tensor, step, cache, pre=None, next_norm=None):
        mixer, ffn = parts["mixer"], parts["ffn"]
        if isinstance(cache, dict):      # a layer with several parts that keep a cache: each gets its own
            cache = cache.get("mixer")
        rt = mixer.rt
        h = NormedInput(x, parts["mixer_norm"], rt.dtype, pre)
        emit = NormEmit.of(parts["ffn_norm"]) if mixer.emits_next_norm and ffn.takes_normed_input else None
        if mixer.emits_next_norm:
            mixer.forward_add(h if mixer.takes_normed_input else h.tensor(), step, cache, x, emit=emit)
        else:
            mixer.forward_add(h if mixer.takes_normed_input else h.tensor(), step, cache, x)
        h = NormedInput(x, parts["ffn_norm"], rt.dtype, emit)
        emit = NormEmit.of(next_norm) if ffn.emits_next_norm else None
        if ffn.emits_next_norm:
            ffn.forward_add(h if ffn.takes_normed_input else h.tensor(), step, x, emit=emit)
        else:
            ffn.forward_add(h if ffn.takes_normed_input else h.tensor(), step, x)
        return emit if emit is not None and emit.filled else None
