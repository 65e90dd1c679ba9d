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
    num_pages: int = 0                 # 0: sized from max_tokens
    max_tokens: int = 8192             # tokens the cache pool holds when num_pages is 0
    max_active_requests: int = 64
    max_batch_tokens: int = 2048       # token budget of one step
    chunk_tokens: int = 512            # largest portion of one prompt in a step
    seed: int = 0xA110ACA              # crates/allpaca-core/src/sampling.rs:5-8
    use_graphs: bool = True            # replay decode-only steps as HIP graphs
    device: str = "cuda:0"

    def validate(self) -> None:
        if self.dtype not in ("bfloat16", "float32"):
            raise ValueError(f"dtype must be 'bfloat16' or 'float32', got {self.dtype!r}")
        for name in ("page_tokens", "max_active_requests", "max_batch_tokens", "chunk_tokens"):
            if getattr(self, name) <= 0:
                raise ValueError(f"{name} must be positive")
