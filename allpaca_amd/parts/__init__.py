from .base import (ARRANGEMENTS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS, POSITION_ENCODINGS, FeedForward,
                   FixedState, Mixer, Norm, NormEmit, NormedInput, PagedKV, Part, PositionEncoding, Runtime, as_normed,
                   build_part, need_kind)
from .spec import BlockSpec, ModelSpec, ParamSpec, PartSpec, PlanEntry
from . import attention, block, embedding, mlp, norm, rope  # noqa: F401  (registers the built-in parts)
from .block import Block

__all__ = ["ARRANGEMENTS", "EMBEDDINGS", "FEED_FORWARDS", "HEADS", "MIXERS", "NORMS", "POSITION_ENCODINGS",
           "FeedForward", "FixedState", "Mixer", "Norm", "PagedKV", "Part", "PositionEncoding", "Runtime",
           "build_part", "need_kind", "NormEmit", "NormedInput", "as_normed", "BlockSpec", "ModelSpec", "ParamSpec", "PartSpec", "PlanEntry", "Block"]
