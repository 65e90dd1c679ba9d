"""Seeded random weights for any described model, and a writer that turns a
configuration and a seed into a model folder (config.json, model.safetensors).

The reference's synthetic model draws uniform values from one generator in a
fixed order (crates/allpaca-core/src/model.rs:5061-5125, 13369-13387); here each
tensor has a generator of its own keyed by (seed, tensor name), so a tensor does
not depend on which others exist or in which order they are made.  Matrices are
N(0, std); norm weights are 1 + N(0, norm_std); a tensor may name its own rule
(`ParamSpec.init`: a bias that starts at zero, a rate that starts at a constant)."""
from __future__ import annotations

import hashlib
import json
import os
from typing import Any, Dict, Mapping, Optional

import torch

from ..parts.spec import ParamSpec
from .safetensors_io import write_safetensors_streamed


def _tensor_seed(seed: int, name: str) -> int:
    h = hashlib.sha256(f"{int(seed)}:{name}".encode()).digest()
    return int.from_bytes(h[:8], "little") & 0x7FFFFFFFFFFFFFFF


def random_tensors(specs: Mapping[str, ParamSpec], seed: int, dtype: torch.dtype, std: float = 0.02,
                   norm_std: float = 0.0, device: str | torch.device = "cpu") -> Dict[str, torch.Tensor]:
    """name -> tensor.  "compute" tensors get `dtype`; norm weights float32; integer tables zeros."""
    out: Dict[str, torch.Tensor] = {}
    dev = torch.device(device)
    for name, ps in specs.items():
        g = torch.Generator(device=dev)
        g.manual_seed(_tensor_seed(seed, name))
        want = stored_dtype(ps, dtype)
        init = ps.init
        if init is None:
            init = {"int32": "zeros", "float32": "ones_plus_normal"}.get(ps.store, "normal")
        if isinstance(init, (int, float)) and not isinstance(init, bool):
            t = torch.full(ps.shape, float(init), dtype=torch.float32, device=dev)
        elif init == "zeros":
            t = torch.zeros(ps.shape, dtype=torch.float32, device=dev)
        elif init == "ones_plus_normal":
            t = torch.ones(ps.shape, dtype=torch.float32, device=dev)
            if norm_std:
                t += norm_std * torch.randn(ps.shape, generator=g, dtype=torch.float32, device=dev)
        elif init == "normal":
            t = torch.randn(ps.shape, generator=g, dtype=torch.float32, device=dev) * std
        else:
            raise ValueError(f"tensor {name!r}: init {init!r} is not 'normal', 'ones_plus_normal', 'zeros' or a number")
        out[name] = t.to(want)
    return out


def stored_dtype(ps: ParamSpec, dtype: torch.dtype) -> torch.dtype:
    return torch.int32 if ps.store == "int32" else torch.float32 if ps.store == "float32" else dtype


def write_model_folder(path: str, config_json: Mapping[str, Any], seed: int, dtype: torch.dtype = torch.float32,
                       std: float = 0.02, norm_std: float = 0.0,
                       overrides: Optional[Mapping[str, torch.Tensor]] = None, keep_tensors: bool = True,
                       device: str | torch.device = "cpu") -> Optional[Dict[str, torch.Tensor]]:
    """Writes `path/config.json` and `path/model.safetensors` for the architecture that
    `config_json` names.  `overrides` replaces tensors by name (tests plant values with it).
    Tensors are made and written one at a time; `keep_tensors=False` returns None instead of all of them (a model
    of many GB is then never held whole in memory); `device`: where the random numbers are drawn (a seed gives
    other values on another kind of device)."""
    from ..models import DecoderModel, describe_model
    _, cfg, spec = describe_model(config_json)
    specs = DecoderModel(spec).param_specs()
    overrides = dict(overrides or {})
    for name, t in overrides.items():
        if name not in specs:
            raise KeyError(f"override {name!r} is not a tensor of this model")
        if tuple(t.shape) != tuple(specs[name].shape):
            raise ValueError(f"override {name!r} has shape {tuple(t.shape)}, needs {tuple(specs[name].shape)}")
    kept: Dict[str, torch.Tensor] = {}

    def make(name: str) -> torch.Tensor:
        want = stored_dtype(specs[name], dtype)
        if name in overrides:
            t = overrides[name].to(want)
        else:
            t = random_tensors({name: specs[name]}, seed, dtype, std, norm_std, device)[name]
        if keep_tensors:
            kept[name] = t.cpu()
        return t

    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(dict(config_json), f, indent=1)
    write_safetensors_streamed(os.path.join(path, "model.safetensors"),
                               [(name, stored_dtype(ps, dtype), tuple(ps.shape)) for name, ps in specs.items()], make,
                               {"format": "pt", "seed": str(seed)})
    return kept if keep_tensors else None
