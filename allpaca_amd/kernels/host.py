"""The host library (`csrc/host/`): its structures and entry points for ctypes.

`ApcMatrix`, `ApcLayer`, `ApcPlanEntry`, `ApcStep` and `ApcTunables` mirror `csrc/host/host.h` field by field."""
from __future__ import annotations

import ctypes
from ctypes import POINTER, Structure, c_char_p, c_float, c_int, c_longlong, c_size_t, c_void_p

from . import lib as _lib


class ApcMatrix(Structure):
    _fields_ = [("data", c_void_p), ("packed", c_int), ("dtype", c_int), ("N", c_int), ("K", c_int),
                ("chunks", c_int), ("ld", c_int)]


class ApcLayer(Structure):
    _fields_ = [("norm1_w", c_void_p), ("norm2_w", c_void_p), ("norm1_eps", c_float), ("norm2_eps", c_float),
                ("w_qkv", ApcMatrix), ("w_o", ApcMatrix), ("H", c_int), ("Hk", c_int), ("d", c_int), ("window", c_int),
                ("scale", c_float), ("rot", c_int), ("cos_sin", c_void_p), ("w_gate", ApcMatrix), ("w_up", ApcMatrix),
                ("w_down", ApcMatrix), ("F", c_int)]


class ApcPlanEntry(Structure):
    _fields_ = [("layer", c_int), ("kv", c_void_p), ("kv_dtype", c_int), ("group", c_int), ("page_tokens", c_int),
                ("writes", c_int)]


STEP_ARRAYS = ("tokens", "positions", "row_seg", "seg_row0", "seg_rows", "seg_pos0", "state_slots", "logit_rows",
               "decode_rows", "tile_row0", "tile_rows")


class ApcStep(Structure):
    _fields_ = ([("T", c_int), ("S", c_int), ("R", c_int), ("n_decode", c_int), ("n_tiles", c_int)]
                + [(name, c_void_p) for name in STEP_ARRAYS]
                + [("n_groups", c_int), ("table", c_void_p * 8), ("table_width", c_int * 8),
                   ("max_decode_context", c_int), ("all_rows_decode", c_int), ("max_prompt_keys", c_int)])


class ApcStepFinding(Structure):
    _fields_ = [("what", c_int), ("entry", c_int), ("value", c_int), ("extra", c_int)]


class ApcPacked(Structure):
    _fields_ = [("T", c_int), ("S", c_int), ("R", c_int), ("n_decode", c_int), ("n_tiles", c_int), ("total", c_int),
                ("off", c_int * 11), ("n_groups", c_int), ("table_off", c_int * 8), ("table_width", c_int * 8),
                ("max_decode_context", c_int), ("max_prompt_keys", c_int), ("max_context", c_int), ("max_rows", c_int)]


class ApcTunables(Structure):
    _fields_ = [("whole_min_pairs", c_int), ("last_block_merges", c_int), ("wide_tiles", c_int),
                ("key_splits_max", c_int), ("key_range_min", c_int), ("force_plain", c_int)]


P, I = c_void_p, c_int
_lib.SIGNATURES["host"].update({
    "apc_host_program_new": [I, I, I, POINTER(ApcMatrix), P, c_float, POINTER(ApcMatrix)],
    "apc_host_program_free": [P],
    "apc_host_program_add_layer": [P, POINTER(ApcLayer)],
    "apc_host_program_add_entry": [P, POINTER(ApcPlanEntry)],
    "apc_host_program_tunables": [P, POINTER(ApcTunables), P, I],
    "apc_host_step_bytes": [P, POINTER(ApcStep)],
    "apc_host_step_begin": [P, POINTER(ApcStep), P, c_size_t, P],
    "apc_host_step_range": [P, I, I],
    "apc_host_step_finish": [P, P],
    "apc_host_step": [P, POINTER(ApcStep), P, c_size_t, P, P],
    "apc_host_residual_offset": [P],
    "apc_host_timing": [P, I],
    "apc_host_timing_report": [P],
    "apc_host_rule_tiled_k_split": [I, I, I],
    "apc_host_rule_decode_parts": [c_longlong, I],
    "apc_host_rule_key_splits": [I, I, I, I, I, I],
    # ---- the cache manager's books
    "apc_pool_new": [I], "apc_pool_free": [P], "apc_pool_alloc": [P], "apc_pool_give_back": [P, I],
    "apc_pool_free_count": [P], "apc_pool_pages": [P], "apc_pool_allocations": [P],
    "apc_pool_held": [P, POINTER(c_int), I], "apc_pool_log_frees": [P, I], "apc_pool_drain": [P, POINTER(c_int), I],
    "apc_cache_new": [I, I, POINTER(c_int), POINTER(c_int), I], "apc_cache_free": [P], "apc_cache_pool": [P, I],
    "apc_cache_admit": [P, c_longlong], "apc_cache_release": [P, c_longlong],
    "apc_cache_reserve": [P, c_longlong, I], "apc_cache_commit": [P, c_longlong, I],
    "apc_cache_truncate": [P, c_longlong, I], "apc_cache_length": [P, c_longlong], "apc_cache_slot": [P, c_longlong],
    "apc_cache_version": [P, c_longlong], "apc_cache_pages_needed": [P, c_longlong, I, POINTER(c_int)],
    "apc_cache_table": [P, c_longlong, I, POINTER(c_int), I], "apc_cache_check": [P], "apc_cache_why": [P],
    # ---- the step packer (array arguments as addresses: numpy arrays' `ctypes.data`)
    "apc_step_prepare": [P, I, I, I, P, P, P, P, P, POINTER(ApcStepFinding)],
    "apc_step_commit": [P, I, P, P],
    "apc_pack_layout": [P, I, P, P, P, I, I, POINTER(ApcPacked)],
    "apc_pack_step": [P, I, P, P, P, P, P, I, I, P, P, I, POINTER(ApcPacked)],
    # ---- the scheduler
    "apc_sched_new": [P, I, I, I, I], "apc_sched_free": [P], "apc_sched_too_large": [P, I, I, POINTER(c_int)],
    "apc_sched_add": [P, c_longlong, I, I, I],
    "apc_sched_plan": [P, POINTER(c_longlong), I, POINTER(c_longlong), POINTER(c_longlong), POINTER(c_int), I,
                       POINTER(c_int)],
    "apc_sched_advance": [P, c_longlong, I], "apc_sched_token": [P, c_longlong], "apc_sched_finish": [P, c_longlong],
    "apc_sched_counts": [P, POINTER(c_int)],
})
_lib.RESTYPES.update({
    "apc_host_program_new": c_void_p, "apc_host_program_free": None, "apc_host_program_tunables": None,
    "apc_host_step_bytes": c_longlong, "apc_host_residual_offset": c_longlong, "apc_host_timing": None,
    "apc_host_timing_report": c_char_p,
    "apc_pool_new": c_void_p, "apc_pool_free": None, "apc_pool_allocations": c_longlong, "apc_pool_log_frees": None,
    "apc_cache_new": c_void_p, "apc_cache_free": None, "apc_cache_pool": c_void_p, "apc_cache_version": c_longlong,
    "apc_cache_why": c_char_p, "apc_sched_new": c_void_p, "apc_sched_free": None,
})

ERRORS = {-10: "the work space is too small for this step", -11: "calls out of order (no step was begun)"}


def load():
    """The host library (built first if need be; the kernel libraries it is linked against are loaded with it)."""
    _lib.load("plain")
    _lib.load("tuned")
    return _lib.load("host")


def check(code: int, what: str) -> None:
    if code in ERRORS:
        raise _lib.KernelError(f"{what}: {ERRORS[code]}")
    _lib.check(code, what)
