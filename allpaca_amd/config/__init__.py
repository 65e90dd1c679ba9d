"""Configuration: the model's config.json (typed per architecture) and the
engine's own options."""
from __future__ import annotations

import json
import os
from typing import Any, Mapping

from .engine import EngineConfig
from .llama import ConfigError, Llama3RopeScaling, LlamaConfig


def read_config_json(model_dir: str) -> dict:
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"{path}: no config.json in the model folder")
    try:
        with open(path) as f:
            d = json.load(f)
    except json.JSONDecodeError as e:
        raise ConfigError(f"{path}: not valid JSON ({e})") from None
    if not isinstance(d, dict):
        raise ConfigError(f"{path}: top level must be an object")
    return d


__all__ = ["ConfigError", "EngineConfig", "Llama3RopeScaling", "LlamaConfig", "read_config_json"]


def preset(name: str) -> dict:
    """A config.json of a known model shape, kept as data under `config/presets/`."""
    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), "presets")
    path = os.path.join(here, name + ".json")
    if not os.path.isfile(path):
        known = sorted(f[:-5] for f in os.listdir(here) if f.endswith(".json"))
        raise ConfigError(f"no preset {name!r}; known: {', '.join(known)}")
    with open(path) as f:
        return json.load(f)
