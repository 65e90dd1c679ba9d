"""Architectures: a name -> (typed configuration, model description) table, and
the one decoder class that runs any description."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Mapping, Tuple

from ..config import ConfigError, read_config_json
from ..parts.spec import ModelSpec
from ..registry import Registry, UnknownName


@dataclass(frozen=True)
class Architecture:
    name: str
    read_config: Callable[[Mapping[str, Any]], Any]   # config.json dict -> typed configuration
    describe: Callable[[Any], ModelSpec]               # typed configuration -> ModelSpec


ARCHITECTURES: Registry = Registry("architecture")


def architecture_of(config_json: Mapping[str, Any]) -> Architecture:
    """By `architectures[0]`, then by `model_type`."""
    names = list(config_json.get("architectures") or [])
    candidates = names[:1] + ([config_json["model_type"]] if config_json.get("model_type") else [])
    for n in candidates:
        if n in ARCHITECTURES:
            return ARCHITECTURES.get(n)
    if not candidates:
        raise ConfigError("config.json names no architecture (keys 'architectures' and 'model_type' are both absent)")
    raise ConfigError(f"config.json names architecture {candidates!r}; known: {', '.join(ARCHITECTURES.names())}")


def describe_model(config_json: Mapping[str, Any]) -> Tuple[Architecture, Any, ModelSpec]:
    arch = architecture_of(config_json)
    cfg = arch.read_config(config_json)
    spec = arch.describe(cfg)
    spec.validate()
    return arch, cfg, spec


from . import llama  # noqa: E402,F401  (registers itself)
from .decoder import DecoderModel, load_model  # noqa: E402

__all__ = ["ARCHITECTURES", "Architecture", "architecture_of", "describe_model", "DecoderModel", "load_model"]
