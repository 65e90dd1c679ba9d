"""What a part is, and the registries parts are chosen from.

A part (mixer, feed-forward, norm, position encoding, embedding, head) is built
from its own sizes and constants only; it never sees a model configuration and
does not know which model it is in.  It names the tensors it wants
(`param_specs`), receives them (`bind`), and computes on the rows it is given.

Interfaces
----------
Norm            forward(x[T,D] float32 residual or activations, out[T,D]) ; forward_rows(x, rows, out)
PositionEncoding  table-driven rotation or any in-place transform of q and k by per-row positions
Mixer           cache_need() -> PagedKV | FixedState | None
                forward_add(h[T,D], step, cache, residual[T,D] float32): residual += mixer(h)
FeedForward     forward_add(h[T,D], step, residual[T,D] float32): residual += ffn(h)
Arrangement     run(block_parts, x, step, cache): one layer on the residual stream x
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Mapping, Optional, Tuple, Union

import torch

from ..registry import Registry
from .spec import ParamSpec, PartSpec

MIXERS: Registry = Registry("mixer")
FEED_FORWARDS: Registry = Registry("feed-forward")
NORMS: Registry = Registry("norm")
POSITION_ENCODINGS: Registry = Registry("position encoding")
ARRANGEMENTS: Registry = Registry("block arrangement")
EMBEDDINGS: Registry = Registry("embedding")
HEADS: Registry = Registry("output head")


# ---- what a mixer needs of the cache manager -------------------------------
@dataclass(frozen=True)
class PagedKV:
    """Keys and values of every position (or of the last `window` positions) in pages."""
    kv_heads: int
    head_dim: int
    window: Optional[int] = None


@dataclass(frozen=True)
class FixedState:
    """Per-request state of fixed size in a slot (zeroed when a request is admitted)."""
    shape: Tuple[int, ...]
    dtype: str = "float32"


CacheNeed = Union[PagedKV, FixedState, None]


@dataclass
class Runtime:
    """Where and how a built model runs."""
    device: torch.device
    dtype: torch.dtype               # activations and 16-bit matrices: torch.bfloat16 or torch.float32
    max_positions: int               # positions the position tables must cover

    @property
    def is_float32(self) -> bool:
        return self.dtype == torch.float32


class Part:
    """Base of every part."""

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {}

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        """Receives the tensors named by `param_specs` (CPU or GPU) and moves what it keeps to `rt.device`."""
        self.rt = rt


class Norm(Part):
    def forward(self, x: torch.Tensor, out: torch.Tensor, rows: Optional[torch.Tensor] = None) -> None:
        raise NotImplementedError


class PositionEncoding(Part):
    """`fused()` returns (rot, cos_sin table) when the encoding is a pairwise rotation
    (i, i + rot/2) that the rotation-and-cache-write kernel can apply; otherwise None and
    `apply` is called on q and k before they are cached."""

    def fused(self):
        return None

    def apply(self, qkv: torch.Tensor, q_off: int, k_off: int, n_heads: int, n_kv_heads: int, head_dim: int,
              positions: torch.Tensor) -> None:
        raise NotImplementedError


class Mixer(Part):
    # True if `forward_add` only launches kernels whose arguments stay valid when the step's device
    # buffers are refilled (nothing read back to the host, no host-side branching on the batch): such a
    # mixer's decode steps can be replayed as a HIP graph
    graph_safe = False

    def cache_need(self) -> CacheNeed:
        return None

    def forward(self, h: torch.Tensor, step, cache) -> torch.Tensor:
        raise NotImplementedError

    def forward_add(self, h: torch.Tensor, step, cache, residual: torch.Tensor) -> None:
        from ..kernels import ops
        ops.add_into(residual, self.forward(h, step, cache))


class FeedForward(Part):
    def forward(self, h: torch.Tensor, step) -> torch.Tensor:
        raise NotImplementedError

    def forward_add(self, h: torch.Tensor, step, residual: torch.Tensor) -> None:
        from ..kernels import ops
        ops.add_into(residual, self.forward(h, step))


def build_part(registry: Registry, spec: PartSpec) -> Part:
    cls = registry.get(spec.kind)
    try:
        return cls(**dict(spec.params))
    except TypeError as e:
        raise TypeError(f"{registry.what} {spec.kind!r}: {e}") from None


def to_device(t: torch.Tensor, rt: Runtime, dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    return t.to(device=rt.device, dtype=dtype or t.dtype).contiguous()
