"""Weights by tensor name: what the model asks for is checked against what the
files hold, and every problem is reported in one error.

Storage rule: a matrix used by matrix products ("compute") is kept in bfloat16
when the run is bfloat16 and the file holds it in 16 bits (float16 is widened to
float32, which is exact); a tensor stored in 32-bit stays in 32-bit; in a
float32 run everything is widened.  Norm weights ("float32") are always held in
float32; integer tables as int32."""
from __future__ import annotations

from typing import Dict, List, Mapping, Optional, Sequence

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
                 ignored_suffixes: tuple = (), aliases: Optional[Mapping[str, Sequence[str]]] = None
                 ) -> Dict[str, torch.Tensor]:
    """CPU tensors for every name in `wanted` (converted by the storage rule).
    Raises one `WeightsError` naming all missing, unexpected and wrongly shaped tensors.
    `forbidden`: names that must not be there (name -> reason), except that a name in `copies` may be there if it
    equals, bit for bit, the tensor `copies[name]`; names with an ending in `ignored_suffixes` are passed over.
    `aliases`: name -> ordered candidates under which the files may hold it; the first that is present is taken, a
    missing tensor is reported with every candidate tried (crates/allpaca-safetensors/src/catalog.rs:117-141), and a
    tensor that is present under two of its names is an error."""
    files = open_model_files(model_dir)
    where: Dict[str, SafetensorsFile] = {}
    other: List[str] = []
    for f in files:
        for name in f.entries:
            if name in where:  # crates/allpaca-safetensors/src/catalog.rs:65-98
                other.append(f"tensor {name} appears in both {where[name].path} and {f.path}")
            where[name] = f
    forbidden = dict(forbidden or {})
    aliases = aliases or {}

    def candidates(name: str) -> List[str]:
        c = list(aliases.get(name, ()))
        return c if name in c else [name] + c

    found: Dict[str, str] = {}        # wanted or forbidden name -> the name the files hold it under
    stands_for: Dict[str, str] = {}   # the other way round
    for name in list(wanted) + [n for n in forbidden if n not in wanted]:
        present = [c for c in candidates(name) if c in where]
        if len(present) > 1:
            other.append(f"tensor {name} is present under more than one of its names: {', '.join(present)}")
        if present:
            found[name] = present[0]
            stands_for[present[0]] = name
    # names that are another spelling of a tensor already found (reported above, not once more as unexpected)
    second_names = {c for name in found for c in candidates(name) if c != found[name]}
    missing, wrong = [], []
    for name, spec in wanted.items():
        if name not in found:
            if not spec.optional:
                tried = [c for c in candidates(name) if c != name]
                missing.append(name + (f" (also tried: {', '.join(tried)})" if tried else ""))
            continue
        held = found[name]
        dt, shape = where[held].entries[held]
        label = name if held == name else f"{held} (for {name})"
        if tuple(shape) != tuple(spec.shape):
            wrong.append((label, shape, spec.shape))
        if spec.store == "int32" and dt not in ("I32", "I64"):
            other.append(f"tensor {label} must be an integer table, the file holds {dt}")
        if spec.store != "int32" and dt in ("I32", "I64"):
            other.append(f"tensor {label} must be floating point, the file holds {dt}")
    unexpected = []
    for held in where:
        name = stands_for.get(held, held)
        if name in wanted and found.get(name) == held:
            continue
        if name in forbidden and found.get(name) == held:
            twin = found.get((copies or {}).get(name))
            if twin in where and where[held].entries[held] == where[twin].entries[twin] and \
                    torch.equal(where[held].tensor(held).view(torch.uint8), where[twin].tensor(twin).view(torch.uint8)):
                continue     # the same matrix stored twice
            other.append(f"tensor {held} must not be present: {forbidden[name]}"
                         + (f" (it is there and differs from {twin})" if twin in where else ""))
        elif any(held.endswith(suffix) for suffix in ignored_suffixes):
            continue
        elif held not in second_names:
            unexpected.append(held)
    if missing or unexpected or wrong or other:
        raise WeightsError(model_dir, sorted(missing), sorted(unexpected), wrong, other)
    out: Dict[str, torch.Tensor] = {}
    for name, spec in wanted.items():
        if name not in found:
            continue
        t = where[found[name]].tensor(found[name])
        out[name] = t.to(target_dtype(spec, t.dtype, run_dtype))  # a copy unless the type already matches
    return out
