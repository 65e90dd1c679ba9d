"""Reading and writing of the safetensors container, on its own terms.

Format (crates/allpaca-safetensors/src/parser.rs:11, 93-160): 8 bytes of
little-endian header length, a JSON header {name: {dtype, shape, data_offsets}}
(`__metadata__` skipped), then the payload.  Files are memory-mapped; a tensor
is a view until it is copied to the GPU."""
from __future__ import annotations

import json
import mmap
import os
import struct
import warnings
from typing import Dict, Iterable, List, Mapping, Tuple

import numpy as np
import torch

MAX_HEADER = 100 * 1024 * 1024  # parser.rs:11

# file dtype -> (torch dtype, bytes per element)
DTYPES = {
    "F32": (torch.float32, 4),
    "BF16": (torch.bfloat16, 2),
    "F16": (torch.float16, 2),
    "I32": (torch.int32, 4),
    "I64": (torch.int64, 8),
}
NAMES = {v[0]: k for k, v in DTYPES.items()}


class SafetensorsError(ValueError):
    pass


class SafetensorsFile:
    """One memory-mapped file: `.entries[name] = (dtype, shape)`, `.tensor(name)`."""

    def __init__(self, path: str):
        self.path = path
        try:
            self._f = open(path, "rb")
        except OSError as e:
            raise SafetensorsError(f"{path}: cannot open ({e.strerror})") from None
        size = os.fstat(self._f.fileno()).st_size
        if size < 8:
            raise SafetensorsError(f"{path}: too short for a safetensors header")
        (hlen,) = struct.unpack("<Q", self._f.read(8))
        if hlen > MAX_HEADER or 8 + hlen > size:
            raise SafetensorsError(f"{path}: header length {hlen} overruns the file ({size} bytes)")
        try:
            header = json.loads(self._f.read(hlen).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise SafetensorsError(f"{path}: header is not valid JSON ({e})") from None
        self._base = 8 + hlen
        self._map = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ) if size > 0 else None
        self.entries: Dict[str, Tuple[str, Tuple[int, ...]]] = {}
        self._spans: Dict[str, Tuple[int, int]] = {}
        for name, info in header.items():
            if name == "__metadata__":
                continue
            dt, shape = info.get("dtype"), tuple(info.get("shape", ()))
            lo, hi = info.get("data_offsets", (0, 0))
            if dt not in DTYPES:
                raise SafetensorsError(f"{path}: tensor {name!r} has unsupported dtype {dt!r} "
                                       f"(supported: {', '.join(DTYPES)})")
            count = int(np.prod(shape, dtype=np.int64)) if shape else 1
            if hi - lo != count * DTYPES[dt][1] or self._base + hi > size or lo < 0:
                raise SafetensorsError(f"{path}: tensor {name!r} spans bytes {lo}..{hi}, which does not fit its "
                                       f"shape {list(shape)} of {dt} or the file")
            self.entries[name] = (dt, shape)
            self._spans[name] = (lo, hi)

    def tensor(self, name: str) -> torch.Tensor:
        """A CPU tensor viewing the mapped bytes (read-only memory: copy before writing)."""
        dt, shape = self.entries[name]
        lo, hi = self._spans[name]
        if hi == lo:
            return torch.empty(shape, dtype=DTYPES[dt][0])
        buf = memoryview(self._map)[self._base + lo : self._base + hi]
        arr = np.frombuffer(buf, dtype=np.uint8)
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")  # torch warns that the mapped bytes are read-only; they are only read
            return torch.from_numpy(arr).view(DTYPES[dt][0]).reshape(shape)

    def close(self) -> None:
        self.entries = {}
        # the map stays alive while tensors view it; nothing to release explicitly


def open_model_files(model_dir: str) -> List[SafetensorsFile]:
    """`model.safetensors`, or the shards of `model.safetensors.index.json`
    (crates/allpaca-safetensors/src/catalog.rs:51-98)."""
    single = os.path.join(model_dir, "model.safetensors")
    index = os.path.join(model_dir, "model.safetensors.index.json")
    if os.path.isfile(index):
        with open(index) as f:
            wm = json.load(f).get("weight_map") or {}
        if not wm:
            raise SafetensorsError(f"{index}: empty weight_map")
        return [SafetensorsFile(os.path.join(model_dir, fn)) for fn in sorted(set(wm.values()))]
    if os.path.isfile(single):
        return [SafetensorsFile(single)]
    others = sorted(f for f in os.listdir(model_dir) if f.endswith(".safetensors")) if os.path.isdir(model_dir) else []
    if len(others) == 1:
        return [SafetensorsFile(os.path.join(model_dir, others[0]))]
    if others:
        raise SafetensorsError(f"{model_dir}: several .safetensors files and no model.safetensors.index.json")
    raise SafetensorsError(f"{model_dir}: no model.safetensors")


def _write_tensor(f, t: torch.Tensor) -> None:
    """The tensor's bytes, straight from its memory (no copy of the whole tensor into a bytes object)."""
    c = t.detach().cpu().contiguous()
    if c.numel():
        f.write(memoryview(c.reshape(-1).view(torch.uint8).numpy()))


def write_safetensors_streamed(path: str, entries, make, metadata: Mapping[str, str] | None = None) -> None:
    """Writes a file whose tensors are made one at a time: `entries` = [(name, torch dtype, shape)] in file order,
    `make(name)` returns the tensor (CPU or GPU) when its turn comes, so a model of many GB is never held whole."""
    header: Dict[str, dict] = {}
    if metadata:
        header["__metadata__"] = dict(metadata)
    off = 0
    for name, dtype, shape in entries:
        if dtype not in NAMES:
            raise SafetensorsError(f"cannot write tensor {name!r} of type {dtype}")
        n = int(np.prod(shape, dtype=np.int64)) * DTYPES[NAMES[dtype]][1] if len(shape) else DTYPES[NAMES[dtype]][1]
        header[name] = {"dtype": NAMES[dtype], "shape": list(shape), "data_offsets": [off, off + n]}
        off += n
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for name, dtype, shape in entries:
            t = make(name)
            if t.dtype != dtype or tuple(t.shape) != tuple(shape):
                raise SafetensorsError(f"tensor {name!r} came as {t.dtype} {list(t.shape)}, announced as {dtype} {list(shape)}")
            _write_tensor(f, t)


def write_safetensors(path: str, tensors: Mapping[str, torch.Tensor], metadata: Mapping[str, str] | None = None) -> None:
    """Writes tensors (CPU or GPU) in the order given."""
    write_safetensors_streamed(path, [(name, t.dtype, tuple(t.shape)) for name, t in tensors.items()],
                               lambda name: tensors[name], metadata)
