"""Seeded random weights for any described model, and a writer that turns a
configuration and a seed into a model folder (config.json, model.safetensors).

The reference's synthetic model draws uniform values from one generator in a
fixed order (crates/allpaca-core/src/model.rs:5061-5125, 13369-13387); here every
element has a number of its own, a hash of (seed, tensor name, index of the
element), so a tensor does not depend on which others exist or in which order
they are made, nor on where it is made: the arithmetic is integer up to one
float32 multiplication, and a seed gives the same bits on the CPU and on the
GPU.  Matrices are N(0, std); norm weights are 1 + N(0, norm_std); a tensor may
name its own rule (`ParamSpec.init`: a bias that starts at zero, a rate that
starts at a constant).  "N" is the sum of four uniform 16-bit numbers, scaled
to unit variance (its tails end at 3.5 deviations)."""
from __future__ import annotations

import hashlib
import json
import os
from typing import Any, Dict, Mapping, Optional

import torch

from ..parts.spec import ParamSpec
from .safetensors_io import write_safetensors_streamed

_M64 = (1 << 64) - 1
_CHUNK = 1 << 25          # elements drawn at a time (a few hundred MB of int64 temporaries)


def _tensor_seed(seed: int, name: str) -> int:
    h = hashlib.sha256(f"{int(seed)}:{name}".encode()).digest()
    return int.from_bytes(h[:8], "little") & 0x7FFFFFFFFFFFFFFF


def _signed(x: int) -> int:
    x &= _M64
    return x - (1 << 64) if x >> 63 else x


def _shr(x: torch.Tensor, n: int) -> torch.Tensor:
    """Logical shift right of int64 (the operator shifts the sign in)."""
    return (x >> n) & ((1 << (64 - n)) - 1)


def unit_normal(base: int, count: int, device: torch.device, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """float32 [count]: element i is a function of (base, i) alone: splitmix64 of base + i * an odd constant, its four
    16-bit pieces added up (mean 131070, variance 4 (2^32 - 1) / 12) and scaled to mean 0 and variance 1."""
    out = torch.empty(count, dtype=torch.float32, device=device) if out is None else out
    scale = float((3.0 / (2 ** 32 - 1)) ** 0.5)
    for lo in range(0, count, _CHUNK):
        n = min(_CHUNK, count - lo)
        i = torch.arange(lo, lo + n, dtype=torch.int64, device=device)
        x = i * _signed(0xD6E8FEB86659FD93) + _signed(base + 0x9E3779B97F4A7C15)      # (wraps modulo 2^64)
        z = (x ^ _shr(x, 30)) * _signed(0xBF58476D1CE4E5B9)
        z = (z ^ _shr(z, 27)) * _signed(0x94D049BB133111EB)
        z = z ^ _shr(z, 31)
        total = (z & 0xFFFF) + (_shr(z, 16) & 0xFFFF) + (_shr(z, 32) & 0xFFFF) + _shr(z, 48)
        out[lo:lo + n] = (total - 131070).to(torch.float32) * scale
    return out


def random_tensors(specs: Mapping[str, ParamSpec], seed: int, dtype: torch.dtype, std: float = 0.02,
                   norm_std: float = 0.0, device: str | torch.device = "cpu") -> Dict[str, torch.Tensor]:
    """name -> tensor.  "compute" tensors get `dtype`; norm weights float32; integer tables zeros."""
    out: Dict[str, torch.Tensor] = {}
    dev = torch.device(device)
    for name, ps in specs.items():
        want = stored_dtype(ps, dtype)
        init = ps.init
        if init is None:
            init = {"int32": "zeros", "float32": "ones_plus_normal"}.get(ps.store, "normal")
        count = 1
        for n in ps.shape:
            count *= int(n)
        if isinstance(init, (int, float)) and not isinstance(init, bool):
            t = torch.full(ps.shape, float(init), dtype=torch.float32, device=dev)
        elif init == "zeros":
            t = torch.zeros(ps.shape, dtype=torch.float32, device=dev)
        elif init == "ones_plus_normal":
            t = torch.ones(ps.shape, dtype=torch.float32, device=dev)
            if norm_std:
                t += unit_normal(_tensor_seed(seed, name), count, dev).view(ps.shape) * float(norm_std)
        elif init == "normal":
            t = unit_normal(_tensor_seed(seed, name), count, dev).view(ps.shape)
            t *= float(std)
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
    the same values wherever)."""
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
