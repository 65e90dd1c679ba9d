"""Loads the kernel libraries with ctypes and declares their entry points.

Every entry point is `extern "C" int apc_*(..., hipStream_t)`; it returns 0, a
hipError_t (> 0) or one of our own codes (< 0).  There is no fallback: if a
library cannot be built or loaded the caller gets `KernelLibraryError`."""
from __future__ import annotations

import ctypes
from typing import Dict

from . import build as _build

P, I, F, Z = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_size_t


class KernelLibraryError(RuntimeError):
    pass


class KernelError(RuntimeError):
    pass


# name -> argument types (the trailing stream included)
SIGNATURES: Dict[str, Dict[str, list]] = {
    "plain": {
        "apc_embed_rows": [P, I, P, P, I, I, I, I, P],
        "apc_embed_rows_tiled": [P, I, P, P, I, I, I, I, P],
        "apc_gather_rows": [P, I, I, P, P, I, I, I, P],
        "apc_rmsnorm_rows": [P, I, I, P, P, F, P, I, I, I, I, P],
        "apc_add_into": [P, I, P, I, I, I, I, P],
        "apc_silu_mul": [P, I, I, P, I, I, I, I, P],
        "apc_rope_kv_write": [P, I, I, I, I, I, I, I, I, I, I, P, P, P, P, I, P, I, I, P],
        "apc_cast": [P, I, P, I, Z, P],
        "apc_gemm_plain": [P, I, I, P, I, I, P, I, I, I, I, I, I, P],
        "apc_paged_attention_plain": [P, I, I, I, P, I, I, I, I, I, I, P, I, I, P, I, P, P, I, F, P],
        "apc_argmax_rows": [P, I, I, I, P, P, P],
        "apc_argmax_rows_no_alloc": [P, I, I, I, P, P],
        "apc_sample_rows": [P, I, I, I, P, P, P, P, P, P, Z, I, P],
        "apc_sample_rows_scratch_kib": [I],
    },
    "tuned": {
        "apc_gemm_bf16": [P, I, P, P, I, I, I, I, I, P],
        "apc_gemm_swiglu_bf16": [P, I, P, P, P, I, I, I, I, P],
        "apc_skinny_gemm_emit_bf16": [P, I, P, P, I, I, I, I, P, P, I, P, P],
        "apc_skinny_gemm_pre_bf16": [P, I, P, I, F, P, P, I, I, I, I, I, P],
        "apc_skinny_swiglu_pre_bf16": [P, I, P, I, F, P, P, P, I, I, I, I, P],
        "apc_skinny_qkv_rope_bf16": [P, I, P, I, F, P, P, I, I, I, I, I, I, P, P, P, P, I, P, I, P],
        "apc_rope_kv_write_bf16": [P, I, I, I, I, I, I, I, I, I, P, P, P, P, I, P, I, P],
        "apc_gemm_splitk_emit_bf16": [P, I, P, P, I, I, I, I, I, P, P, P, I, P, P],
        "apc_gemm_pre_bf16": [P, I, P, I, F, P, P, P, I, I, I, I, I, P],
        "apc_gemm_splitk_qkv_rope_bf16": [P, I, P, I, F, P, P, I, I, I, I, I, I, P, P, P, P, I, P, I, I, P, P],
        "apc_gemm_splitk_pre_bf16": [P, I, P, I, F, P, P, P, I, I, I, I, I, I, P, P],
        "apc_gemm_splitk_bf16": [P, I, P, P, P, I, I, I, I, I, I, P, P],
        "apc_gemm_direct_k_split": [I, I, I],
        "apc_gemm_direct_emit_parts": [P, I, P, I, I, I, I],
        "apc_gemm_direct_emit_bf16": [P, I, P, P, I, I, I, I, P, P, I, P, I, P, P],
        "apc_skinny_gemm_bf16": [P, I, P, P, I, I, I, I, I, P],
        "apc_skinny_swiglu_bf16": [P, I, P, P, P, I, I, I, I, P],
        "apc_attention_prefill_bf16": [P, I, I, P, I, I, I, I, P, I, P, I, P, P, P, P, I, I, I, F, I, I, P, P],
        "apc_attention_decode_bf16": [P, I, I, P, I, I, I, I, I, P, I, P, I, P, P, P, I, F, I, I, P, P, P],
        "apc_attention_decode_last_fits": [I, I, I, I],
        "apc_attention_decode_whole_fits": [I, I, I],
        "apc_attention_prefill_tile_rows": [],
        "apc_attention_prefill_wide_takes": [I, I, I, I],
    },
    "bench": {
        "apc_probe_read": [P, Z, P, I, I, I, P],
        "apc_probe_mfma": [I, P, I, P],
    },
}

# The host library's entry points take structures (declared in `kernels/host.py`, which fills this in) and some
# return something other than an int.
SIGNATURES["host"] = {}
RESTYPES: Dict[str, object] = {}

_loaded: Dict[str, "Library"] = {}

ERRORS = {-1: "bad argument (shape or stride the kernel does not accept)", -2: "size not supported by this kernel",
          -3: "more rows than the entry point that allocates nothing has room for"}


class KernelTimer:
    """Event timers around every call of an entry point while it is active (`with lib.timing() as t:`): for a pass
    of its own beside the measured one, as the reference keeps its per-kernel timers out of the measured run
    (one forward in 16 is timed with events and bucketed per kernel, crates/allpaca-hip/src/lib.rs:7776-7790).
    `records`: (entry point, its arguments of C type int in order, start event, end event)."""

    def __init__(self):
        self.records = []

    def totals(self) -> Dict[str, dict]:
        """entry point -> {"calls", "us", "args": integer arguments of its calls in order}; waits for the GPU."""
        import torch
        torch.cuda.synchronize()
        out: Dict[str, dict] = {}
        for name, ints, e0, e1 in self.records:
            t = out.setdefault(name, {"calls": 0, "us": 0.0, "args": []})
            t["calls"] += 1
            t["us"] += e0.elapsed_time(e1) * 1e3
            t["args"].append(ints)
        return out


_timer = None
# entry points that launch nothing (questions about sizes): never timed
NOT_KERNELS = {"apc_attention_decode_whole_fits", "apc_attention_decode_last_fits", "apc_attention_prefill_tile_rows",
               "apc_attention_prefill_wide_takes",
               "apc_gemm_direct_k_split", "apc_gemm_direct_emit_parts", "apc_sample_rows_scratch_kib"}


class timing:
    def __enter__(self) -> KernelTimer:
        global _timer
        _timer = KernelTimer()
        return _timer

    def __exit__(self, *exc) -> None:
        global _timer
        _timer = None


class _EntryPoint:
    __slots__ = ("name", "fn", "int_at")

    def __init__(self, name: str, fn, argtypes):
        self.name, self.fn = name, fn
        self.int_at = tuple(i for i, t in enumerate(argtypes) if t is I)

    def __call__(self, *args):
        if _timer is None or self.name in NOT_KERNELS:
            return self.fn(*args)
        import torch
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        code = self.fn(*args)
        e1.record()
        _timer.records.append((self.name, tuple(int(args[i]) for i in self.int_at), e0, e1))
        return code


class Library:
    """The entry points of one kernel library as attributes (each may be timed, see `timing`)."""

    def __init__(self, cdll: ctypes.CDLL, path: str):
        self._cdll, self.path = cdll, path


def load(name: str) -> Library:
    """The library `name`, built first if it is missing or stale."""
    lib = _loaded.get(name)
    if lib is not None:
        return lib
    try:
        path = _build.build(name)
    except _build.KernelBuildError as e:
        raise KernelLibraryError(f"kernel library '{name}' is not available: {e}") from None
    try:
        cdll = ctypes.CDLL(path)
    except OSError as e:
        raise KernelLibraryError(f"cannot load {path}: {e}") from None
    lib = Library(cdll, path)
    for fn, args in SIGNATURES[name].items():
        try:
            f = getattr(cdll, fn)
        except AttributeError:
            raise KernelLibraryError(f"{path} lacks entry point {fn}") from None
        f.argtypes = args
        f.restype = RESTYPES.get(fn, I)
        setattr(lib, fn, _EntryPoint(fn, f, args) if name != "host" else f)
    _loaded[name] = lib
    return lib


def check(code: int, what: str) -> None:
    if code == 0:
        return
    if code < 0:
        raise KernelError(f"{what}: {ERRORS.get(code, f'error {code}')}")
    raise KernelError(f"{what}: HIP error {code}")
