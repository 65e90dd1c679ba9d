"""Options of the engine itself (not of a model)."""
from __future__ import annotations

from dataclasses import dataclass


@dataclass
class EngineConfig:
    """`page_tokens` and `chunk_tokens` carry the reference's names
    (`kv.page_tokens`, `prefill.chunk_tokens`, crates/allpaca-types/src/config.rs:326-336,
    671-683; `engine.max_active_requests` 386-403)."""
    dtype: str = "bfloat16"            # "bfloat16" | "float32"
    page_tokens: int = 16
    num_pages: int = 0                 # pages of the cache pool; 0: sized from max_tokens
    max_tokens: int = 0                # tokens the cache pool holds when num_pages is 0; 0 too: sized from memory
    # With neither given, the pool takes `kv_bytes`, or, if that is 0, the device memory that is free once the
    # weights are loaded minus `kv_reserve_bytes` (room for a step's activations, logits and workspaces; 0: worked out
    # from `max_batch_tokens`, `max_active_requests` and the model's widths, `Engine.reserve_bytes`); never more than
    # every one of `max_active_requests` requests at the model's longest context needs (the reference's budget is
    # `kv.vram_bytes`, crates/allpaca-core/src/engine.rs:8651-8680).  "Free" is what the device reports when the
    # engine is built: processes that share a GPU each see the same figure, so give each its `kv_bytes` or `max_tokens`.
    kv_bytes: int = 0
    kv_reserve_bytes: int = 0
    max_active_requests: int = 64
    max_batch_tokens: int = 2048       # token budget of one step
    chunk_tokens: int = 512            # largest portion of one prompt in a step
    # rows of a tile of the bfloat16 matrix products: a step that overshoots a multiple of it by a few rows has its
    # last prompt portion cut back to the multiple (0: never)
    step_row_tile: int = 128
    seed: int = 0xA110ACA              # crates/allpaca-core/src/sampling.rs:5-8
    use_graphs: bool = True            # replay decode-only steps as HIP graphs
    device: str = "cuda:0"

    def validate(self) -> None:
        if self.dtype not in ("bfloat16", "float32"):
            raise ValueError(f"dtype must be 'bfloat16' or 'float32', got {self.dtype!r}")
        for name in ("page_tokens", "max_active_requests", "max_batch_tokens", "chunk_tokens"):
            if getattr(self, name) <= 0:
                raise ValueError(f"{name} must be positive")
        for name in ("num_pages", "max_tokens", "kv_bytes", "kv_reserve_bytes"):
            if getattr(self, name) < 0:
                raise ValueError(f"{name} must not be negative")
