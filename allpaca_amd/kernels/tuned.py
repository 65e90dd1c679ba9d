"""Checked wrappers of the bfloat16 MFMA kernels (library `tuned`).  Each checks what the kernel
assumes.  Matrix products take weights in the tiled layout (`packing.PackedWeight`), which only
matrices of a width that is a multiple of 8 get (`ops.prepare_matrix`): other widths stay row-major
and run on the plain kernel.  Attention returns False for sizes it does not take (a page size that is
no multiple of 8, a head size that is no multiple of 16 or above 256) and the caller runs the plain
kernel: never a wrong result."""
from __future__ import annotations

import math
from typing import Optional

import torch

from . import lib as _lib
from . import ops as _ops
from .packing import PackedWeight

MANY_ROWS_SPLIT_MAX = 1024   # up to here the tiled kernel may cut K into slices to get enough blocks
SKINNY_MAX_ROWS = 16     # the streaming kernel: up to one 16-row tile of activations
SPLITK_MAX_ROWS = 128    # the tiled kernel with K cut into slices: 17..128 rows


def _k_split(M: int, N: int, K: int) -> int:
    """Slices of K for the split kernel with 17..128 rows: about 240 blocks in all (measured best at the shapes of 3B
    and 8B models: 32 column tiles in 6-8 slices, 48 in 4-5, 224 whole), at least 4 K-steps of 64 each."""
    blocks = -(-N // 128) * -(-M // 128)
    s = max(1, min(12, round(240 / blocks)))
    return max(1, min(s, K // 256))


def _k_split_many_rows(M: int, N: int, K: int) -> int:
    """Slices of K for 129..1024 rows: a matrix with few output columns gives the 128 x 128 tiles too few blocks
    for 256 compute units (o_proj and down of an 8B model at 512 rows: 128), and slicing K, at the price of writing
    and adding float32 partial sums, was measured faster up to about 200 blocks (down, 4096 x 14336, 256 rows: 150
    us whole, 52 us in 4 slices); with more outputs than K and 150 blocks or more it was not."""
    blocks = -(-N // 128) * -(-M // 128)
    if blocks <= 56:
        s = 5
    elif blocks <= 68:
        s = 4
    elif blocks <= 88:
        s = 3
    elif blocks <= 208 and not (blocks >= 150 and N > K):
        s = 2
    else:
        s = 1
    return max(1, min(s, K // 256))


def _tiled_k_split(M: int, N: int, K: int) -> int:
    """Slices of K on the tiled kernel for M rows (1: K in one piece)."""
    if M <= SPLITK_MAX_ROWS:
        return _k_split(M, N, K)
    return _k_split_many_rows(M, N, K) if M <= MANY_ROWS_SPLIT_MAX else 1


# The chip these rules and the kernels' launch plans were measured on (`csrc/host/rules.h`, `gemm_direct_bf16.hip`:
# rounds of 256 blocks over 8 XCDs; `attention_wide_bf16.hip`: 160 KiB of LDS a compute unit).
CHIP_UNITS = 256
CHIP_LDS_BYTES = 160 * 1024
_chips_checked: set = set()


def check_chip(device: torch.device) -> None:
    """Says so, once per device, if the GPU is not the one the dispatch rules were measured on: the results stay
    right (no kernel assumes the counts for correctness), the cuts may be badly chosen."""
    import warnings
    key = (device.type, device.index)
    if device.type != "cuda" or key in _chips_checked:
        return
    _chips_checked.add(key)
    prop = torch.cuda.get_device_properties(device)
    units = getattr(prop, "multi_processor_count", CHIP_UNITS)
    lds = getattr(prop, "shared_memory_per_block_optin", 0) or getattr(prop, "shared_memory_per_block", 0)
    if units != CHIP_UNITS or (lds and lds < CHIP_LDS_BYTES):
        warnings.warn(f"{prop.name}: {units} compute units and {lds} bytes of LDS a block; the bfloat16 kernels' dispatch "
                      f"rules were measured on {CHIP_UNITS} units with {CHIP_LDS_BYTES} bytes and may be badly tuned here")


def _aligned(*ts: torch.Tensor) -> bool:
    return all(t.data_ptr() % 16 == 0 for t in ts)


def _act_ok(a: torch.Tensor) -> bool:
    return (a.dtype == torch.bfloat16 and a.shape[1] % 8 == 0 and _ops._rows(a, "a") % 8 == 0 and _aligned(a))


def gemm_bf16(a: torch.Tensor, w: PackedWeight, out: torch.Tensor, accumulate: bool = False) -> None:
    """out = a . w^T (bfloat16 or float32 out), or out += a . w^T (float32 out); w in the tiled layout."""
    _ops._gpu(a, w.data, out)
    M, K = a.shape
    N = w.N
    if not (w.K == K):
        raise ValueError(f"gemm: a is [*, {K}] but w is {w.shape}")
    if not (out.shape == (M, N)):
        raise ValueError(f"gemm: out must be [{M}, {N}], got {tuple(out.shape)}")
    _ops._need(not accumulate or out.dtype == torch.float32, "gemm: accumulation needs a float32 destination")
    _ops._need(out.dtype in (torch.bfloat16, torch.float32), "gemm: out must be bfloat16 or float32")
    _ops._need(w.data.is_contiguous() and w.data.shape[0] * 16 >= N and w.data.shape[1] * 32 >= K,
               "gemm: the tiled weight does not cover [N, K]")
    if not _act_ok(a):
        raise ValueError("gemm_bf16: activations must be bfloat16 rows of a width and stride that are multiples "
                         "of 8, 16-byte aligned")
    lda, ldc = _ops._rows(a, "a"), _ops._rows(out, "out")
    mode = 2 if accumulate else (0 if out.dtype == torch.bfloat16 else 1)
    L = _lib.load("tuned")
    if M > SKINNY_MAX_ROWS:
        # more than 1,024 rows: the product of many rows says itself whether it wants K in two slices
        ks = _tiled_k_split(M, N, K) if M <= MANY_ROWS_SPLIT_MAX else L.apc_gemm_direct_k_split(M, N, K)
        if ks > 1:
            ws = torch.empty(ks * M * N, dtype=torch.float32, device=a.device)
            _lib.check(L.apc_gemm_splitk_bf16(a.data_ptr(), lda, w.data.data_ptr(), 0, out.data_ptr(), ldc, M, N, K,
                                              mode, ks, ws.data_ptr(), _ops._stream()), "gemm_splitk_bf16")
            return
    fn = L.apc_skinny_gemm_bf16 if M <= SKINNY_MAX_ROWS else L.apc_gemm_bf16
    _lib.check(fn(a.data_ptr(), lda, w.data.data_ptr(), out.data_ptr(), ldc, M, N, K, mode, _ops._stream()),
               "gemm_bf16")


def swiglu_bf16(h: torch.Tensor, wg: PackedWeight, wu: PackedWeight, out: torch.Tensor) -> None:
    """out[t, f] = silu(h . Wg[f]) * (h . Wu[f]); Wg, Wu in the tiled layout."""
    _ops._gpu(h, wg.data, wu.data, out)
    M, K = h.shape
    F = out.shape[1]
    if not (wg.shape == (F, K) and wu.shape == (F, K)):
        raise ValueError(f"swiglu: weights must both be [{F}, {K}]")
    _ops._need(out.shape[0] == M and out.dtype == torch.bfloat16, "swiglu: out must be bfloat16 [rows, F]")
    if not _act_ok(h):
        raise ValueError("swiglu_bf16: activations must be bfloat16 rows of a width and stride that are multiples "
                         "of 8, 16-byte aligned")
    lda, ldc = _ops._rows(h, "h"), _ops._rows(out, "out")
    L = _lib.load("tuned")
    ks = _tiled_k_split(M, 2 * F, K) if M > SKINNY_MAX_ROWS else 1
    if ks > 1:
        ws = torch.empty(2 * ks * M * F, dtype=torch.float32, device=h.device)
        _lib.check(L.apc_gemm_splitk_bf16(h.data_ptr(), lda, wg.data.data_ptr(), wu.data.data_ptr(), out.data_ptr(), ldc,
                                          M, F, K, 3, ks, ws.data_ptr(), _ops._stream()), "gemm_splitk_bf16")
        return
    fn = L.apc_skinny_swiglu_bf16 if M <= SKINNY_MAX_ROWS else L.apc_gemm_swiglu_bf16
    _lib.check(fn(h.data_ptr(), lda, wg.data.data_ptr(), wu.data.data_ptr(), out.data_ptr(), ldc, M, F, K,
                  _ops._stream()), "swiglu_bf16")


def gemm_emit_bf16(a: torch.Tensor, w: PackedWeight, residual: torch.Tensor, g: torch.Tensor):
    """residual += a . w^T, and for the RMS norm with weight g that reads the residual next: the row
    bfloat16(residual * g) and sums of residual^2 per row and group of columns.  Returns (raw [M, N], ss) or None,
    with nothing done, for sizes no kernel takes.  ss is [16, ceil(N/16) rounded up to 4] from the streaming kernel
    (up to 16 rows) and [M, ceil(N/256)] from the tiled kernel with K in slices; the products below take what the
    same number of rows gives."""
    _ops._gpu(a, w.data, residual, g)
    M, K = a.shape
    N = w.N
    if (not _act_ok(a) or residual.dtype != torch.float32 or g.dtype != torch.float32 or g.numel() != N
            or not g.is_contiguous()):
        return None
    if not (w.K == K and residual.shape == (M, N)):
        raise ValueError(f"gemm: a [{M}, {K}], w {w.shape}, residual {tuple(residual.shape)}")
    L = _lib.load("tuned")
    lda, ldc = _ops._rows(a, "a"), _ops._rows(residual, "residual")
    if M > MANY_ROWS_SPLIT_MAX:
        # the product of many rows: its own epilogue leaves the row, or with K in two slices the kernel that adds them
        # (sums of squares per tile of columns, or per 1,024 columns)
        parts = L.apc_gemm_direct_emit_parts(a.data_ptr(), lda, residual.data_ptr(), ldc, M, N, K)
        if not parts:
            return None
        raw = torch.empty((M, N), dtype=torch.bfloat16, device=a.device)
        ss = torch.empty((M, parts), dtype=torch.float32, device=a.device)
        ks = L.apc_gemm_direct_k_split(M, N, K)
        ws = torch.empty(ks * M * N, dtype=torch.float32, device=a.device) if ks > 1 else None
        _lib.check(L.apc_gemm_direct_emit_bf16(a.data_ptr(), lda, w.data.data_ptr(), residual.data_ptr(), ldc, M, N, K,
                                               g.data_ptr(), raw.data_ptr(), N, ss.data_ptr(), parts,
                                               ws.data_ptr() if ws is not None else 0, _ops._stream()),
                   "gemm_direct_emit_bf16")
        return raw, ss
    if M > SKINNY_MAX_ROWS:   # the tiled kernel: only where K is cut into slices (the finishing kernel leaves the row)
        ks = _tiled_k_split(M, N, K)
        if ks == 1:
            # With K in one piece the product's own epilogue would have to do it; measured at 2,048 rows that costs
            # 20-27 us a product, more than the norm's kernel (10 us) that it would save.
            return None
        raw = torch.empty((M, N), dtype=torch.bfloat16, device=a.device)
        ss = torch.empty((M, -(-N // 256)), dtype=torch.float32, device=a.device)
        ws = torch.empty(ks * M * N, dtype=torch.float32, device=a.device)
        _lib.check(L.apc_gemm_splitk_emit_bf16(a.data_ptr(), lda, w.data.data_ptr(), residual.data_ptr(), ldc, M, N, K,
                                               ks, ws.data_ptr(), g.data_ptr(), raw.data_ptr(), N, ss.data_ptr(),
                                               _ops._stream()), "gemm_splitk_emit_bf16")
        return raw, ss
    raw = torch.empty((M, N), dtype=torch.bfloat16, device=a.device)
    ss = torch.empty((16, -(-(-(-N // 16)) // 4) * 4), dtype=torch.float32, device=a.device)
    _lib.check(L.apc_skinny_gemm_emit_bf16(a.data_ptr(), lda, w.data.data_ptr(), residual.data_ptr(), ldc, M, N, K,
                                           g.data_ptr(), raw.data_ptr(), N, ss.data_ptr(), _ops._stream()),
               "skinny_gemm_emit_bf16")
    return raw, ss


def _pre_ok(raw: torch.Tensor, ss: torch.Tensor, K: int) -> bool:
    return (raw.shape[0] <= SKINNY_MAX_ROWS and _act_ok(raw) and ss.dtype == torch.float32 and ss.is_contiguous()
            and tuple(ss.shape) == (16, -(-(-(-K // 16)) // 4) * 4))


def _pre_tiled(raw: torch.Tensor, ss: torch.Tensor, eps: float, w, wu, out: torch.Tensor, n_cols: int, mode: int) -> bool:
    """The same on the tiled kernel (more than 16 rows), K in slices or in one piece: ss is [M, parts] with up to
    256 sums of squares a row (what the tiled kernels leave: a part per 256 or per 128 columns)."""
    M, K = raw.shape
    if not (M > SKINNY_MAX_ROWS and _act_ok(raw) and ss.dtype == torch.float32 and ss.is_contiguous()
            and ss.dim() == 2 and ss.shape[0] == M and 1 <= ss.shape[1] <= 256):
        return False
    n_mats = 2 if wu is not None else 1
    ks = _tiled_k_split(M, n_cols * n_mats, K)
    L = _lib.load("tuned")
    wu_ptr = wu.data.data_ptr() if wu is not None else 0
    if ks == 1:
        _lib.check(L.apc_gemm_pre_bf16(raw.data_ptr(), _ops._rows(raw, "raw"), ss.data_ptr(), ss.shape[1], float(eps),
                                       w.data.data_ptr(), wu_ptr, out.data_ptr(), _ops._rows(out, "out"), M, n_cols, K,
                                       mode, _ops._stream()), "gemm_pre_bf16")
        return True
    ws = torch.empty(n_mats * ks * M * n_cols, dtype=torch.float32, device=raw.device)
    _lib.check(L.apc_gemm_splitk_pre_bf16(raw.data_ptr(), _ops._rows(raw, "raw"), ss.data_ptr(), ss.shape[1], float(eps),
                                          w.data.data_ptr(), wu_ptr, out.data_ptr(), _ops._rows(out, "out"), M, n_cols,
                                          K, mode, ks, ws.data_ptr(), _ops._stream()), "gemm_splitk_pre_bf16")
    return True


def gemm_pre_bf16(raw: torch.Tensor, ss: torch.Tensor, eps: float, w: PackedWeight, out: torch.Tensor) -> bool:
    """out = (raw . w^T) / sqrt(sum(ss) / K + eps) for a row that `gemm_emit_bf16` left: the product of the
    normalised row.  False, with nothing done, for sizes the kernel does not take."""
    _ops._gpu(raw, ss, w.data, out)
    M, K = raw.shape
    if out.dtype not in (torch.bfloat16, torch.float32):
        return False
    if not (w.K == K and out.shape == (M, w.N)):
        raise ValueError(f"gemm: raw [{M}, {K}], w {w.shape}, out {tuple(out.shape)}")
    if M > SKINNY_MAX_ROWS:
        return _pre_tiled(raw, ss, eps, w, None, out, w.N, 0 if out.dtype == torch.bfloat16 else 1)
    if not _pre_ok(raw, ss, K):
        return False
    L = _lib.load("tuned")
    _lib.check(L.apc_skinny_gemm_pre_bf16(raw.data_ptr(), _ops._rows(raw, "raw"), ss.data_ptr(), -(-K // 16), float(eps),
                                          w.data.data_ptr(), out.data_ptr(), _ops._rows(out, "out"), M, w.N, K,
                                          0 if out.dtype == torch.bfloat16 else 1, _ops._stream()),
               "skinny_gemm_pre_bf16")
    return True


def qkv_rope_bf16(a: torch.Tensor, pre, w: PackedWeight, q_out: torch.Tensor, n_heads: int, n_kv_heads: int,
                  head_dim: int, cos_sin: torch.Tensor, positions: torch.Tensor, row_seg: torch.Tensor,
                  block_table: torch.Tensor, cache: torch.Tensor, page_tokens: int) -> bool:
    """q, k, v in one product that also rotates q and k (whole heads) and writes k and v into the pages; rotated q
    goes to the first n_heads * head_dim columns of q_out.  Up to 16 rows: the streaming kernel (head size a
    multiple of 32); more rows: the tiled kernel where it cuts K into slices, in its finishing kernel (256 a
    multiple of the head size).  `a`: the normalised rows, or with `pre` = (ss, eps) the row that
    `gemm_emit_bf16` left.  False, with nothing done, for sizes neither takes."""
    _ops._gpu(a, w.data, q_out, cos_sin, positions, row_seg, block_table, cache)
    M, K = a.shape
    H, Hk, d = n_heads, n_kv_heads, head_dim
    N = (H + 2 * Hk) * d
    few = M <= SKINNY_MAX_ROWS
    if not (_act_ok(a) and q_out.dtype == torch.bfloat16 and cache.dtype == torch.bfloat16):
        return False
    if few and not (d % 32 == 0 and q_out.stride(0) % 4 == 0 and q_out.data_ptr() % 8 == 0):
        return False
    ks = 1 if few else _tiled_k_split(M, N, K)
    if not few and (ks == 1 or 256 % d or d % 2):
        return False
    ss, eps = None, 0.0
    if pre is not None:
        ss, eps = pre
        if few and not _pre_ok(a, ss, K):
            return False
        if not few and not (ss.dtype == torch.float32 and ss.is_contiguous() and ss.dim() == 2 and ss.shape[0] == M
                            and 1 <= ss.shape[1] <= 256):
            return False
    if not (w.K == K and w.N == N and q_out.shape[0] == M and q_out.shape[1] >= H * d):
        raise ValueError(f"qkv: a [{M}, {K}], w {w.shape}, {H}+2*{Hk} heads of {d}, q_out {tuple(q_out.shape)}")
    _ops._need(cos_sin.dtype == torch.float32 and cos_sin.is_contiguous() and tuple(cos_sin.shape[1:]) == (2, d // 2),
               "cos/sin table must be float32 [positions, 2, head_dim/2]")
    if not (cache.dim() == 5 and cache.is_contiguous() and tuple(cache.shape[1:]) == (2, Hk, page_tokens, d)):
        raise ValueError(f"cache must be [pages, 2, {Hk}, {page_tokens}, {d}], got {tuple(cache.shape)}")
    _ops._need(block_table.dim() == 2 and block_table.dtype == torch.int32 and block_table.is_contiguous(),
               "block table must be contiguous int32 [segments, blocks]")
    L = _lib.load("tuned")
    ss_ptr = ss.data_ptr() if ss is not None else 0
    if few:
        _lib.check(L.apc_skinny_qkv_rope_bf16(
            a.data_ptr(), _ops._rows(a, "a"), ss_ptr, -(-K // 16) if ss is not None else 0, float(eps), w.data.data_ptr(),
            q_out.data_ptr(), _ops._rows(q_out, "q_out"), M, K, H, Hk, d, cos_sin.data_ptr(),
            _ops._i32(positions, M, "positions"), _ops._i32(row_seg, M, "row_seg"), block_table.data_ptr(),
            block_table.shape[1], cache.data_ptr(), page_tokens, _ops._stream()), "skinny_qkv_rope_bf16")
        return True
    ws = torch.empty(ks * M * N, dtype=torch.float32, device=a.device)
    _lib.check(L.apc_gemm_splitk_qkv_rope_bf16(
        a.data_ptr(), _ops._rows(a, "a"), ss_ptr, ss.shape[1] if ss is not None else 0, float(eps), w.data.data_ptr(),
        q_out.data_ptr(), _ops._rows(q_out, "q_out"), M, K, H, Hk, d, cos_sin.data_ptr(),
        _ops._i32(positions, M, "positions"), _ops._i32(row_seg, M, "row_seg"), block_table.data_ptr(),
        block_table.shape[1], cache.data_ptr(), page_tokens, ks, ws.data_ptr(), _ops._stream()),
        "gemm_splitk_qkv_rope_bf16")
    return True


def swiglu_pre_bf16(raw: torch.Tensor, ss: torch.Tensor, eps: float, wg: PackedWeight, wu: PackedWeight,
                    out: torch.Tensor) -> bool:
    """SwiGLU of the normalised row, from what `gemm_emit_bf16` left (see `gemm_pre_bf16`)."""
    _ops._gpu(raw, ss, wg.data, wu.data, out)
    M, K = raw.shape
    F = out.shape[1]
    if out.dtype != torch.bfloat16:
        return False
    if not (wg.shape == (F, K) and wu.shape == (F, K) and out.shape[0] == M):
        raise ValueError(f"swiglu: weights must both be [{F}, {K}]")
    if M > SKINNY_MAX_ROWS:
        return _pre_tiled(raw, ss, eps, wg, wu, out, F, 3)
    if not _pre_ok(raw, ss, K):
        return False
    L = _lib.load("tuned")
    _lib.check(L.apc_skinny_swiglu_pre_bf16(raw.data_ptr(), _ops._rows(raw, "raw"), ss.data_ptr(), -(-K // 16),
                                            float(eps), wg.data.data_ptr(), wu.data.data_ptr(), out.data_ptr(),
                                            _ops._rows(out, "out"), M, F, K, _ops._stream()), "skinny_swiglu_pre_bf16")
    return True


def _decode_parts(pairs: int, span: int) -> int:
    """Ranges that the decode kernel cuts the keys of every row into (four to a block, one per wave): as many blocks
    a (row, kv head) pair as keep the launch at one block a compute unit or under, and no range under 64 keys.  The
    kernel sizes a row's ranges from the row's own length, so the count depends on the step's shape alone.  Measured at
    8B shapes (32 heads over 8, heads of 128), 1 to 16 rows over 512 to 8,192 keys, ranges of 64 to 512 keys: the
    fastest choice was in every case the shortest range whose launch fits the chip once (8 rows over 2,063 keys: 256
    blocks 18.9 us, 320 blocks 21.4 us, 192 blocks 20.6 us; over 8,192 keys: 256 blocks 53.3 us, 512 blocks 54.6 us,
    1,024 blocks 56.5 us)."""
    per_pair = max(1, CHIP_UNITS // max(1, pairs))
    return max(1, min(WHOLE_WAVES * per_pair, -(-span // 64)))


# Keys of a range of the decode kernel, the same for every row and counted from position 0, instead of the rule above
# (0: the rule): for measurements and tests.
KEYS_PER_PART = 0


# From how many (row, kv head) pairs on a decode step's attention runs as one block per pair that finishes its heads
# itself (no partial results through memory, no second kernel): the pairs alone then give every compute unit work
# (measured at the shapes of an 8B model: 7-15 % faster from 32 rows on, slower with 16).
WHOLE_MIN_PAIRS = 256
WHOLE_WAVES = 4   # waves of such a block (NW in attention_bf16.hip)


# With fewer pairs: the blocks of a pair leave one partial result each and the one that finishes last adds them (no
# second kernel), where the sizes allow; False: partial results per wave and a kernel that merges them.
LAST_BLOCK_MERGES = True
# Portions whose tiles of 128 rows are mostly whole (heads of 128 or 64, pages of a power of two from 16 on) run on the kernel
# that takes such a tile a block (attention_wide_bf16.hip); False sends every portion to the kernels of 64-row blocks.
WIDE_TILES = True
_counters: dict = {}
# Ranges that the keys of a tile of prompt rows are cut into: never more (0 sends a tile's keys to one block always),
# and the keys a range must keep
KEY_SPLITS_MAX = 8
KEY_RANGE_MIN = 2048


def _key_splits(step, n_heads: int, window: int) -> int:
    """Into how many ranges of keys the 128-row attention kernel cuts every tile of this step: a block per (tile, head)
    leaves compute units idle when a step has few tiles (a chunk of 512 prompt tokens at 32 heads: 128 blocks for 256
    units), so the keys are shared out until the chip has a block a unit, as long as a range keeps KEY_RANGE_MIN keys
    (measured at 8B shapes, 512 rows: 1.2 times as fast at 4,096 keys, 1.56 at 32,768, a loss at 2,048: a block's
    start and the kernel that adds the ranges cost a few tiles of 64 keys), or half as many while the chip stays at
    most half full (a block alone on its compute unit and its neighbours' runs at the pace of its own chain of loads:
    128 rows over 2,048 keys in 2 ranges 1.27 times as fast, over 4,096 keys in 4 ranges 1.9 times).  1: no cutting."""
    blocks = step.n_tiles * n_heads
    pos0 = getattr(step, "host_pos0", None)
    rows = getattr(step, "host_rows", None)
    if not KEY_SPLITS_MAX or blocks <= 0 or not pos0 or not rows:
        return 1
    keys = max([p + n for p, n in zip(pos0, rows) if n > 1] or [0])     # of the longest prompt in the step
    if window:
        keys = min(keys, window + 128)
    few = min(keys // max(1, KEY_RANGE_MIN // 2), 128 // blocks)
    return max(1, min(KEY_SPLITS_MAX, 256 // blocks, max(keys // KEY_RANGE_MIN, few)))


def _pair_counters(device: torch.device, pairs: int) -> torch.Tensor:
    """Zeroed int32 counters, one per (row, kv head tile), that live as long as the process: a call leaves them zero
    again, and a replayed graph keeps pointing at them.  Grown by allocating anew; the old ones stay (graphs)."""
    key = (device.type, device.index if device.index is not None else torch.cuda.current_device())
    have = _counters.setdefault(key, [])
    if not have or have[-1].numel() < pairs:
        have.append(torch.zeros(max(1024, pairs), dtype=torch.int32, device=device))
    return have[-1]


def attention_bf16(q: torch.Tensor, q_off: int, out: torch.Tensor, n_heads: int, n_kv_heads: int, head_dim: int,
                   cache: torch.Tensor, page_tokens: int, block_table: torch.Tensor, step, window: int = 0,
                   scale: Optional[float] = None) -> bool:
    """Attention of a whole step: single-row segments on the split-key decode kernel, longer segments on the
    tiled prefill kernel.  Returns False (nothing done) if the sizes are not ones these kernels take."""
    _ops._gpu(q, out, cache, block_table)
    ldq, ldo = _ops._rows(q, "attention q"), _ops._rows(out, "attention out")
    T = q.shape[0]
    if scale is not None and not scale > 0:
        return False
    if (head_dim % 16 or head_dim > 256 or page_tokens % 8 or ldq % 8 or q_off % 8 or not _aligned(q, cache)
            or q.dtype != torch.bfloat16 or cache.dtype != torch.bfloat16 or out.dtype != torch.bfloat16):
        return False
    _ops._need(q_off + n_heads * head_dim <= q.shape[1], "attention: q heads exceed the row")
    _ops._need(out.shape == (T, n_heads * head_dim), "attention out must be [rows, heads*head_dim]")
    _ops._need(n_heads % n_kv_heads == 0, "heads must be a multiple of kv heads")
    if not (cache.dim() == 5 and cache.is_contiguous()
            and tuple(cache.shape[1:]) == (2, n_kv_heads, page_tokens, head_dim)):
        raise ValueError(f"cache must be [pages, 2, {n_kv_heads}, {page_tokens}, {head_dim}], got {tuple(cache.shape)}")
    _ops._need(block_table.dim() == 2 and block_table.dtype == torch.int32 and block_table.is_contiguous(),
               "block table must be contiguous int32 [segments, blocks]")
    _ops._need(step.positions.numel() >= T and step.row_seg.numel() >= T, "step rows differ from q rows")
    sc = (1.0 / math.sqrt(head_dim)) if scale is None else float(scale)
    L = _lib.load("tuned")
    stream = _ops._stream()
    if step.n_tiles:
        # (only the kernel of 128-row blocks cuts keys into ranges: no room is taken for the others)
        wide = WIDE_TILES and L.apc_attention_prefill_wide_takes(head_dim, page_tokens, step.n_tiles, T - step.n_decode_rows)
        splits = _key_splits(step, n_heads, window) if wide else 1
        parts = (torch.empty(splits * T * n_heads * (head_dim + 2), dtype=torch.float32, device=q.device)
                 if splits > 1 else None)
        _lib.check(L.apc_attention_prefill_bf16(
            q.data_ptr(), ldq, q_off, out.data_ptr(), ldo, n_heads, n_kv_heads, head_dim, cache.data_ptr(),
            page_tokens, block_table.data_ptr(), block_table.shape[1], step.positions.data_ptr(),
            step.row_seg.data_ptr(), step.tile_row0.data_ptr(), step.tile_rows.data_ptr(), step.n_tiles,
            (T - step.n_decode_rows) if WIDE_TILES else 0, int(window), sc, splits, T,
            parts.data_ptr() if parts is not None else 0, stream), "attention_prefill_bf16")
    if step.n_decode_rows:
        n = step.n_decode_rows
        span = min(step.max_decode_context, window) if window else step.max_decode_context
        rows = step.decode_rows.data_ptr() if step.decode_rows is not None else 0
        pairs = n * n_kv_heads * -(-(n_heads // n_kv_heads) // 16)
        n_parts = -(-step.max_decode_context // KEYS_PER_PART) if KEYS_PER_PART else _decode_parts(pairs, span)
        # (rows so short that one block's waves take a pair's ranges need no partial results either)
        if ((pairs >= WHOLE_MIN_PAIRS or n_parts <= WHOLE_WAVES)
                and L.apc_attention_decode_whole_fits(n_heads, n_kv_heads, head_dim)):
            _lib.check(L.apc_attention_decode_bf16(
                q.data_ptr(), ldq, q_off, out.data_ptr(), ldo, n, n_heads, n_kv_heads, head_dim, cache.data_ptr(),
                page_tokens, block_table.data_ptr(), block_table.shape[1], step.positions.data_ptr(),
                step.row_seg.data_ptr(), rows, int(window), sc, 0, 0, 0, 0, stream), "attention_decode_bf16 (whole)")
            return True
        kw = KEYS_PER_PART
        if LAST_BLOCK_MERGES and L.apc_attention_decode_last_fits(n_heads, n_kv_heads, head_dim, n_parts):
            # one partial result a block; the block of a (row, kv head) that finishes last adds them: one launch
            nz = -(-n_parts // WHOLE_WAVES)
            ws = torch.empty(n * n_heads * nz * (head_dim + 2), dtype=torch.float32, device=q.device)
            _lib.check(L.apc_attention_decode_bf16(
                q.data_ptr(), ldq, q_off, out.data_ptr(), ldo, n, n_heads, n_kv_heads, head_dim, cache.data_ptr(),
                page_tokens, block_table.data_ptr(), block_table.shape[1], step.positions.data_ptr(),
                step.row_seg.data_ptr(), rows, int(window), sc, kw, n_parts, ws.data_ptr(),
                _pair_counters(q.device, pairs).data_ptr(), stream), "attention_decode_bf16 (last block merges)")
            return True
        ws = torch.empty(n * n_heads * n_parts * (head_dim + 2), dtype=torch.float32, device=q.device)
        _lib.check(L.apc_attention_decode_bf16(
            q.data_ptr(), ldq, q_off, out.data_ptr(), ldo, n, n_heads, n_kv_heads, head_dim, cache.data_ptr(),
            page_tokens, block_table.data_ptr(), block_table.shape[1], step.positions.data_ptr(),
            step.row_seg.data_ptr(), rows, int(window), sc, kw, n_parts, ws.data_ptr(), 0, stream),
            "attention_decode_bf16")
    return True
