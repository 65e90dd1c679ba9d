"""The one decoder: it runs whatever a `ModelSpec` describes.

Embedding -> the plan's entries in order (each runs a block against its own or a
borrowed cache) -> final norm on the rows whose logits are wanted -> head.  The
residual stream is float32 [T, D] throughout.  Nothing here knows an
architecture's name."""
from __future__ import annotations

from typing import Dict, List, Mapping, Optional

import torch

from ..config import read_config_json
from ..parts import EMBEDDINGS, HEADS, NORMS, Block, Runtime, build_part
from ..parts.base import CacheNeed
from ..parts.spec import ModelSpec, ParamSpec
from ..weights.loader import load_tensors


class DecoderModel:
    def __init__(self, spec: ModelSpec):
        spec.validate()
        self.spec = spec
        self.embedding = build_part(EMBEDDINGS, spec.embedding)
        self.blocks: List[Block] = [Block(b) for b in spec.blocks]
        self.final_norm = build_part(NORMS, spec.final_norm)
        self.head = build_part(HEADS, spec.head)
        self.rt: Optional[Runtime] = None

    # ---- weights -----------------------------------------------------------
    def param_specs(self) -> Dict[str, ParamSpec]:
        out: Dict[str, ParamSpec] = {}
        for name, ps in self.embedding.param_specs().items():
            out[self.spec.embedding.weight_prefix + name] = ps
        for b in self.blocks:
            out.update(b.param_specs())
        for name, ps in self.final_norm.param_specs().items():
            out[self.spec.final_norm.weight_prefix + name] = ps
        for name, ps in self.head.param_specs().items():
            out[self.spec.head.weight_prefix + name] = ps
        return out

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        self.rt = rt

        def local(prefix: str, part) -> Dict[str, torch.Tensor]:
            return {n: tensors[prefix + n] for n in part.param_specs() if prefix + n in tensors}

        self.embedding.bind(local(self.spec.embedding.weight_prefix, self.embedding), rt)
        for b in self.blocks:
            b.bind(tensors, rt)
        self.final_norm.bind(local(self.spec.final_norm.weight_prefix, self.final_norm), rt)
        if getattr(self.head, "tied", False):
            self.head.bind({}, rt, shared=self.embedding.weight)
        else:
            self.head.bind(local(self.spec.head.weight_prefix, self.head), rt)

    # ---- cache needs, one per plan entry -------------------------------------
    def cache_needs(self) -> List[CacheNeed]:
        """What each plan entry needs of the cache manager: None (it borrows, or keeps nothing), one need (only the
        part in the role "mixer" keeps something: the cache view goes to the arrangement as it is), or a dict
        role -> need (the arrangement gets a dict role -> view)."""
        needs: List[CacheNeed] = []
        for e in self.spec.plan:
            asked = {} if e.cache_of is not None else self.blocks[e.block].cache_needs()
            needs.append(None if not asked else asked["mixer"] if list(asked) == ["mixer"] else asked)
        return needs

    # ---- one step ------------------------------------------------------------
    def forward(self, step, caches) -> Optional[torch.Tensor]:
        """`step`: the batch on the device (tokens, positions, segments); `caches[i]`: the
        cache view of plan entry i.  Returns float32 logits [wanted rows, vocab], or None."""
        x = self.embed(step)
        self.run_plan(x, step, caches, 0, len(self.spec.plan), None)
        return self.logits(x, step)

    # The same in three pieces, for callers that record the step's launches in more than one graph.
    def embed(self, step) -> torch.Tensor:
        """The float32 residual stream [rows, hidden] of the step's tokens."""
        x = torch.empty((step.n_rows, self.spec.hidden_size), dtype=torch.float32, device=self.rt.device)
        self.embedding.forward(step.tokens, x)
        return x

    def run_plan(self, x: torch.Tensor, step, caches, lo: int, hi: int, left):
        """Plan entries lo .. hi-1 on the stream x.  `left`: what entry lo-1 left for entry lo's first norm (or
        None); returns what entry hi-1 left for entry hi's."""
        plan = self.spec.plan
        for i in range(lo, hi):
            nxt = self.blocks[plan[i + 1].block].first_norm() if i + 1 < len(plan) else None
            left = self.blocks[plan[i].block].run(x, step, caches[i], pre=left, next_norm=nxt)
        return left

    def logits(self, x: torch.Tensor, step) -> Optional[torch.Tensor]:
        R = step.n_logit_rows
        if R == 0:
            return None
        rt = self.rt
        h = torch.empty((R, self.spec.hidden_size), dtype=rt.dtype, device=rt.device)
        self.final_norm.forward(x, h, rows=step.logit_rows)
        logits = torch.empty((R, self.spec.vocab_size), dtype=torch.float32, device=rt.device)
        self.head.forward(h, logits)
        return logits


def load_model(model_dir: str, dtype: torch.dtype, device: torch.device | str = "cuda:0",
               max_positions: Optional[int] = None, beyond_configured_positions: bool = False):
    """Model folder -> (typed configuration, bound DecoderModel).  The class of the model is
    chosen by config.json.  `max_positions`: positions the run is set up for (position tables), at most the
    configuration's own limit unless `beyond_configured_positions` (the formulas hold at any position, and the
    reference does not read `max_position_embeddings`; a replay of given tokens may go past it)."""
    from . import describe_model
    arch, cfg, spec = describe_model(read_config_json(model_dir))
    model = DecoderModel(spec)
    tensors = load_tensors(model_dir, model.param_specs(), dtype, spec.forbidden, spec.copies, spec.ignored_suffixes,
                           spec.aliases)
    positions = max_positions or spec.max_positions
    if not beyond_configured_positions:
        positions = min(positions, spec.max_positions)
    rt = Runtime(torch.device(device), dtype, positions)
    model.bind(tensors, rt)
    return cfg, model
