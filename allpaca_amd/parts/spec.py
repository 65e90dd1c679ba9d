"""Descriptions of a model as data: which part stands where, with which
parameters, and in which order layers run.  An architecture turns its
configuration into a `ModelSpec`; everything below works from the spec and
never asks which architecture it came from."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Mapping, Optional, Tuple


@dataclass(frozen=True)
class PartSpec:
    """A part chosen by name from its registry, with its sizes and constants."""
    kind: str
    params: Mapping[str, Any] = field(default_factory=dict)
    weight_prefix: str = ""          # added to the block's prefix, e.g. "self_attn."


@dataclass(frozen=True)
class BlockSpec:
    """One layer: parts by role, and the arrangement that wires them.
    The pre-norm arrangement uses roles mixer_norm, mixer, ffn_norm, ffn."""
    arrangement: str
    parts: Mapping[str, PartSpec]
    weight_prefix: str               # e.g. "model.layers.3."


@dataclass(frozen=True)
class PlanEntry:
    """One execution of a block.  `cache_of` names an earlier plan entry whose
    cache this execution reads instead of writing one of its own."""
    block: int
    cache_of: Optional[int] = None


@dataclass(frozen=True)
class ParamSpec:
    """A tensor a part wants from the weight file.
    store: "compute" (a matrix used by matrix products: bfloat16 or float32 as
    the run asks, float32 if the file holds it in 32-bit), "float32" (kept in
    32-bit whatever the file holds: norm weights), "int32" (integer tables)."""
    shape: Tuple[int, ...]
    store: str = "compute"
    optional: bool = False
    alias_of: Optional[str] = None   # full name of another tensor to use when this one is absent by design
    # How random weights are drawn for this tensor: "normal" (N(0, std)), "ones_plus_normal" (1 + N(0, norm_std): a
    # norm's weight), "zeros", or a number (that constant: a bias, a decay rate).  None: by `store`, "normal" for
    # "compute", "ones_plus_normal" for "float32", "zeros" for "int32".
    init: Any = None


@dataclass
class ModelSpec:
    hidden_size: int
    vocab_size: int
    max_positions: int
    embedding: PartSpec
    blocks: List[BlockSpec]
    plan: List[PlanEntry]
    final_norm: PartSpec
    head: PartSpec
    # tensors that must NOT be in the file (a tied head's own matrix): name -> reason
    forbidden: Dict[str, str] = field(default_factory=dict)
    # ... unless they are a copy, bit for bit, of the tensor they stand for (writers that store a tied matrix twice):
    # name -> name of the tensor it must equal
    copies: Dict[str, str] = field(default_factory=dict)
    # endings of tensor names that are no parameters and are passed over (buffers some writers store)
    ignored_suffixes: tuple = ()
    # other names under which a file may hold a tensor: name -> ordered candidates (the name itself among them);
    # the first candidate that the files hold is taken
    aliases: Dict[str, List[str]] = field(default_factory=dict)
    # axes of a token's position that the position encodings read: 1 (the place in the request), or more, and then a
    # step carries int32 [rows, axes] beside the places (`StepInfo.position_axes`, given per request in `Entry.positions`)
    position_axes: int = 1

    def validate(self) -> None:
        for i, e in enumerate(self.plan):
            if not (0 <= e.block < len(self.blocks)):
                raise ValueError(f"plan[{i}] names block {e.block}, the model has {len(self.blocks)}")
            if e.cache_of is not None and not (0 <= e.cache_of < i):
                raise ValueError(f"plan[{i}].cache_of = {e.cache_of} must name an earlier plan entry")
            if e.cache_of is not None and self.plan[e.cache_of].cache_of is not None:
                raise ValueError(f"plan[{i}].cache_of names an entry that itself borrows a cache")
