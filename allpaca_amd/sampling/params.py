"""Request options and results, with the reference's names and defaults
(`GenerationParams`, crates/allpaca-types/src/generation.rs:3-80)."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional


@dataclass
class GenerationParams:
    max_tokens: int = 32          # 0 is taken as 1 (crates/allpaca-core/src/engine.rs:3194)
    temperature: float = 0.8      # <= 1e-5: greedy
    top_k: int = 40               # 0: off
    top_p: float = 0.95           # outside [0, 1): off
    seed: Optional[int] = None    # None: the engine's seed
    stop_token_ids: List[int] = field(default_factory=list)

    def __post_init__(self):
        if self.max_tokens <= 0:
            self.max_tokens = 1
        if self.top_k < 0:
            raise ValueError("top_k must be >= 0")

    @property
    def greedy(self) -> bool:
        return self.temperature <= 1e-5


SamplingParams = GenerationParams  # the same thing under the name other engines use


class FinishReason:
    STOP = "stop"
    LENGTH = "length"


@dataclass
class TokenEvent:
    request_id: int
    token_id: int
    finish_reason: Optional[str] = None
    prompt_tokens: int = 0


@dataclass
class GenerationOutput:
    token_ids: List[int]
    prompt_tokens: int
    completion_tokens: int
    finish_reason: str
    timing: Optional[dict] = None     # seconds: queue, ttft, itl (see `Request.timing`)
