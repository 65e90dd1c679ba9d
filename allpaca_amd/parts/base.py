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
# A need says what it wants kept per request and in what shape; the cache manager and the cache's device memory
# work from `kind`, `page_shape` / `slot_shape` and `dtype` alone, so a mixer may bring a need of its own (a latent
# vector per position, keys without values, state in another element type): a frozen dataclass with these members.
# Plan entries whose needs are equal share a group (a pool of pages of its own and one block table per request, or
# one tensor of slots).
#   kind = "pages":  page_shape(page_tokens) -> the shape of one page of one layer; `window` (None: every position is
#                    kept; n: pages that the last n positions no longer reach are given back during the request);
#                    dtype: None (the run's cache element type) or a name ("float32", "bfloat16", "int32")
#   kind = "slot":   slot_shape() -> the shape of one request's state in one layer, zeroed at admission; dtype as above
@dataclass(frozen=True)
class PagedKV:
    """Keys and values of every position (or of the last `window` positions) in pages: keys [kv_head][slot][d],
    values [kv_head][d][slot] (the same count of elements, see the attention kernels)."""
    kv_heads: int
    head_dim: int
    window: Optional[int] = None
    kind = "pages"
    dtype = None

    def page_shape(self, page_tokens: int) -> Tuple[int, ...]:
        return (2, self.kv_heads, page_tokens, self.head_dim)


@dataclass(frozen=True)
class FixedState:
    """Per-request state of fixed size in a slot (zeroed when a request is admitted)."""
    shape: Tuple[int, ...]
    dtype: str = "float32"
    kind = "slot"

    def slot_shape(self) -> Tuple[int, ...]:
        return tuple(self.shape)


CacheNeed = Any   # PagedKV, FixedState, a need of the mixer's own with the members above, or None


def need_kind(need) -> Optional[str]:
    """"pages", "slot" or None (no cache); raises for an object that is no cache need."""
    if need is None:
        return None
    kind = getattr(need, "kind", None)
    if kind == "pages" and callable(getattr(need, "page_shape", None)):
        return kind
    if kind == "slot" and callable(getattr(need, "slot_shape", None)):
        return kind
    raise TypeError(f"{need!r} is no cache need: it must have kind 'pages' with page_shape(page_tokens) or kind "
                    f"'slot' with slot_shape()")


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
    # True if the part only launches kernels whose arguments stay valid when the step's device buffers are refilled
    # (nothing read back to the host, no host-side branching on the batch's content).  Decode-only steps are replayed
    # as a HIP graph only if every part of the model says so: a part that plans on the host (rows gathered per expert
    # from a routing result, a loop over segments) would otherwise be replayed with the first batch's plan.
    graph_safe = False

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {}

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        """Receives the tensors named by `param_specs` (CPU or GPU) and moves what it keeps to `rt.device`."""
        self.rt = rt

    def native_desc(self):
        """What the compiled plan executor (`engine/native.py`, `csrc/host/exec.cpp`) needs to run this part itself: a
        dict of the part's bound tensors and constants under the names the executor knows for the part's kind, or
        None (the default) for a part it does not know.  A model runs on the executor only if all its parts and
        arrangements answer; otherwise its steps are walked in Python, part by part."""
        return None


class Norm(Part):
    def forward(self, x: torch.Tensor, out: torch.Tensor, rows: Optional[torch.Tensor] = None) -> None:
        raise NotImplementedError

    def rms_params(self):
        """(weight, eps) if this norm is x / sqrt(mean(x^2) + eps) * weight, which the products around it can
        fold in; None for any other norm."""
        return None


class NormEmit:
    """What a product that adds into the residual leaves for the RMS norm that reads the residual next: the row
    bfloat16(x * weight) and sums of x^2, from which that norm's first product gets the product of the normalised
    row without a kernel for the norm.  Made by an arrangement for a part that sets `emits_next_norm`; the part
    passes it to `ops.linear(..., accumulate=True, emit=...)`.  Unfilled, it means nothing."""

    def __init__(self, norm: "Norm"):
        self.norm = norm
        self.weight, self.eps = norm.rms_params()
        self.raw: Optional[torch.Tensor] = None
        self.ss: Optional[torch.Tensor] = None

    @staticmethod
    def of(norm: Optional["Norm"]) -> Optional["NormEmit"]:
        return NormEmit(norm) if norm is not None and norm.rms_params() is not None else None

    @property
    def filled(self) -> bool:
        return self.raw is not None


class NormedInput:
    """The normalised input of a part, not computed yet.  An arrangement hands it to a part that sets
    `takes_normed_input`; the part's first product goes through `linear` / `swiglu`, which use what the
    product before the norm left for it (`pre`, a filled `NormEmit`) and otherwise normalise first (`tensor()`)."""

    def __init__(self, x: torch.Tensor, norm: Norm, dtype: torch.dtype, pre: Optional[NormEmit] = None):
        self.x, self.norm, self.dtype = x, norm, dtype
        self.shape, self.device = x.shape, x.device
        self.pre = pre if pre is not None and pre.filled and pre.norm is norm else None
        self._h: Optional[torch.Tensor] = None

    def tensor(self) -> torch.Tensor:
        if self._h is None:
            self._h = torch.empty(self.x.shape, dtype=self.dtype, device=self.x.device)
            self.norm.forward(self.x, self._h)
        return self._h

    def linear(self, w, out: torch.Tensor) -> None:
        from ..kernels import ops
        p = self.pre
        if p is None or self._h is not None or not ops.linear_pre(p.raw, p.ss, p.eps, w, out):
            ops.linear(self.tensor(), w, out)

    def product(self, op) -> bool:
        """For a part with a fused first product of its own: `op(a, pre)` is called with the row that the product
        before the norm left and pre = (ss, eps) if there is one, otherwise with the normalised tensor and
        pre = None.  `op` returns False if it has done nothing; the part then goes through `linear`."""
        p = self.pre
        if p is not None and self._h is None:
            return bool(op(p.raw, (p.ss, p.eps)))
        return bool(op(self.tensor(), None))

    def swiglu(self, w_gate_up, out: torch.Tensor) -> None:
        from ..kernels import ops
        p = self.pre
        if p is None or self._h is not None or not ops.swiglu_pre(p.raw, p.ss, p.eps, w_gate_up, out):
            ops.swiglu(self.tensor(), w_gate_up, out)


def as_normed(h) -> "NormedInput":
    """A part's input as a `NormedInput`, whether the arrangement gave one or a finished tensor."""
    return h if isinstance(h, NormedInput) else _Finished(h)


class _Finished(NormedInput):
    def __init__(self, h: torch.Tensor):
        self.x, self.norm, self.dtype, self.pre = None, None, h.dtype, None
        self.shape, self.device = h.shape, h.device
        self._h = h


class PositionEncoding(Part):
    """`fused()` returns (rot, cos_sin table) when the encoding is a pairwise rotation
    (i, i + rot/2) that the rotation-and-cache-write kernel can apply; otherwise None and
    `apply` is called on q and k before they are cached."""

    def fused(self):
        return None

    def apply(self, qkv: torch.Tensor, q_off: int, k_off: int, n_heads: int, n_kv_heads: int, head_dim: int,
              positions: torch.Tensor) -> None:
        """`positions`: int32 [rows], or [rows, axes] for a model whose spec asks for more than one position axis."""
        raise NotImplementedError


class Mixer(Part):
    # True if `forward_add` takes its input as a `NormedInput` (see there) instead of a tensor
    takes_normed_input = False
    # True if `forward_add` takes `emit=` (a `NormEmit` or None) for its product into the residual
    emits_next_norm = False
    def cache_need(self) -> CacheNeed:
        return None

    def forward(self, h: torch.Tensor, step, cache) -> torch.Tensor:
        raise NotImplementedError

    def forward_add(self, h: torch.Tensor, step, cache, residual: torch.Tensor) -> None:
        from ..kernels import ops
        ops.add_into(residual, self.forward(h, step, cache))


class FeedForward(Part):
    takes_normed_input = False
    emits_next_norm = False

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
