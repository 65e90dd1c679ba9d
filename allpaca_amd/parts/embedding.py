"""Token embedding (a row copy, no scale: crates/allpaca-core/src/model.rs:8301-8311)
and the output head (logits = h W^T in float32 for the rows that ask,
crates/allpaca-core/src/model.rs:8781-8791)."""
from __future__ import annotations

from typing import Dict, Mapping, Optional

import torch

from ..kernels import ops
from .base import EMBEDDINGS, HEADS, Part, Runtime, to_device
from .spec import ParamSpec


@EMBEDDINGS.register("token_table")
class TokenEmbedding(Part):
    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int):
        self.V, self.D = int(vocab_size), int(hidden_size)

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {"weight": ParamSpec((self.V, self.D))}

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        self.rt = rt
        self.weight = ops.prepare_matrix(to_device(tensors["weight"], rt), rt.dtype)

    def forward(self, tokens: torch.Tensor, out: torch.Tensor) -> None:
        ops.embed_rows(self.weight, tokens, out)

    def native_desc(self):
        return {"kind": "token_table", "weight": self.weight} if type(self) is TokenEmbedding else None


@HEADS.register("linear")
class LinearHead(Part):
    """`tied`: the head uses the embedding matrix and owns no tensor."""
    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int, tied: bool = False):
        self.V, self.D, self.tied = int(vocab_size), int(hidden_size), bool(tied)

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {} if self.tied else {"weight": ParamSpec((self.V, self.D))}

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime, shared: Optional[torch.Tensor] = None) -> None:
        self.rt = rt
        self.weight = shared if self.tied else ops.prepare_matrix(to_device(tensors["weight"], rt), rt.dtype)
        if self.weight is None:
            raise ValueError("a tied head needs the embedding matrix")

    def forward(self, h: torch.Tensor, out: torch.Tensor) -> None:
        ops.linear(h, self.weight, out)

    def native_desc(self):
        return {"kind": "linear", "weight": self.weight} if type(self) is LinearHead else None
