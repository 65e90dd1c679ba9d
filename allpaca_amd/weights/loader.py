"""Weights by tensor name: what the model asks for is checked against what the
files hold, and every problem is reported in one error.

Storage rule: a matrix used by matrix products ("compute") is kept in bfloat16
when the run is bfloat16 and the file holds it in 16 bits (float16 is widened to
float32, which is exact); a tensor stored in 32-bit stays in 32-bit; in a
float32 run everything is widened.  Norm weights ("float32") are always held in
float32; integer tables as int32."""
from __future__ import annotations

from typing import Dict, List, Mapping, Optional

import torch

from ..parts.spec import ParamSpec
from .safetensors_io import SafetensorsFile, open_model_files


class WeightsError(ValueError):
    """Lists `missing`, `unexpected`, `wrong_shape` (name, got, expected) and `other` problems."""

    def __init__(self, where: str, missing=(), unexpected=(), wrong_shape=(), other=()):
        self.missing, self.unexpected = list(missing), list(unexpected)
        self.wrong_shape, self.other = list(wrong_shape), list(other)
        lines = [f"{where}: the weights do not match the model"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        for name, got, want in self.wrong_shape:
            lines.append(f"  wrong shape: {name} is {list(got)}, the configuration needs {list(want)}")
        for msg in self.other:
            lines.append(f"  {msg}")
        super().__init__("\n".join(lines))


def target_dtype(spec: ParamSpec, stored: torch.dtype, run_dtype: torch.dtype) -> torch.dtype:
    if spec.store == "int32":
        return torch.int32
    if spec.store == "float32" or run_dtype == torch.float32:
        return torch.float32
    return torch.bfloat16 if stored == torch.bfloat16 else torch.float32


def load_tensors(model_dir: str, wanted: Mapping[str, ParamSpec], run_dtype: torch.dtype,
                 forbidden: Optional[Mapping[str, str]] = None, copies: Optional[Mapping[str, str]] = None,
                 ignored_suffixes: tuple = ()) -> Dict[str, torch.Tensor]:
    """CPU tensors for every name in `wanted` (converted by the storage rule).
    Raises one `WeightsError` naming all missing, unexpected and wrongly shaped tensors.
    `forbidden`: names that must not be there (name -> reason), except that a name in `copies` may be there if it
    equals, bit for bit, the tensor `copies[name]`; names with an ending in `ignored_suffixes` are passed over."""
    files = open_model_files(model_dir)
    where: Dict[str, SafetensorsFile] = {}
    other: List[str] = []
    for f in files:
        for name in f.entries:
            if name in where:  # crates/allpaca-safetensors/src/catalog.rs:65-98
                other.append(f"tensor {name} appears in both {where[name].path} and {f.path}")
            where[name] = f
    forbidden = dict(forbidden or {})
    missing, wrong = [], []
    for name, spec in wanted.items():
        if name not in where:
            if not spec.optional:
                missing.append(name)
            continue
        dt, shape = where[name].entries[name]
        if tuple(shape) != tuple(spec.shape):
            wrong.append((name, shape, spec.shape))
        if spec.store == "int32" and dt not in ("I32", "I64"):
            other.append(f"tensor {name} must be an integer table, the file holds {dt}")
        if spec.store != "int32" and dt in ("I32", "I64"):
            other.append(f"tensor {name} must be floating point, the file holds {dt}")
    unexpected = []
    for name in where:
        if name in wanted:
            continue
        if name in forbidden:
            twin = (copies or {}).get(name)
            if twin in where and where[name].entries[name] == where[twin].entries[twin] and \
                    torch.equal(where[name].tensor(name).view(torch.uint8), where[twin].tensor(twin).view(torch.uint8)):
                continue     # the same matrix stored twice
            other.append(f"tensor {name} must not be present: {forbidden[name]}"
                         + (f" (it is there and differs from {twin})" if twin in where else ""))
        elif any(name.endswith(suffix) for suffix in ignored_suffixes):
            continue
        else:
            unexpected.append(name)
    if missing or unexpected or wrong or other:
        raise WeightsError(model_dir, sorted(missing), sorted(unexpected), wrong, other)
    out: Dict[str, torch.Tensor] = {}
    for name, spec in wanted.items():
        if name not in where:
            continue
        t = where[name].tensor(name)
        out[name] = t.to(target_dtype(spec, t.dtype, run_dtype))  # a copy unless the type already matches
    return out
