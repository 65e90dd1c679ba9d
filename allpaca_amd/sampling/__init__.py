from .params import FinishReason, GenerationOutput, GenerationParams, SamplingParams, TokenEvent

__all__ = ["FinishReason", "GenerationOutput", "GenerationParams", "SamplingParams", "TokenEvent"]
