"""Checked wrappers of the bfloat16 MFMA kernels (library `tuned`).  Each checks what the
kernel assumes; a size a kernel does not take (a width that is no multiple of 8, a page size
that is no multiple of 8, a head size that is no multiple of 16 or above 256) goes to the
plain kernel of the same operation instead, never to a wrong result."""
from __future__ import annotations

import math
from typing import Optional

import torch

from . import lib as _lib
from . import ops as _ops

SKINNY_MAX_ROWS = 64


def _aligned(*ts: torch.Tensor) -> bool:
    return all(t.data_ptr() % 16 == 0 for t in ts)


def _mfma_ok(a: torch.Tensor, w: torch.Tensor) -> bool:
    K = a.shape[1]
    return (K % 8 == 0 and _ops._rows(a, "a") % 8 == 0 and _ops._rows(w, "w") % 8 == 0 and _aligned(a, w)
            and a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16)


def gemm_bf16(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, accumulate: bool = False) -> None:
    """out = a . w^T (bfloat16 or float32 out), or out += a . w^T (float32 out)."""
    _ops._gpu(a, w, out)
    M, K = a.shape
    N = w.shape[0]
    _ops._need(w.shape[1] == K, f"gemm: a is [*, {K}] but w is {tuple(w.shape)}")
    _ops._need(out.shape == (M, N), f"gemm: out must be [{M}, {N}], got {tuple(out.shape)}")
    _ops._need(not accumulate or out.dtype == torch.float32, "gemm: accumulation needs a float32 destination")
    if not _mfma_ok(a, w) or out.dtype not in (torch.bfloat16, torch.float32):
        return _ops.gemm_plain(a, w, out, accumulate)
    lda, ldw, ldc = _ops._rows(a, "a"), _ops._rows(w, "w"), _ops._rows(out, "out")
    mode = 2 if accumulate else (0 if out.dtype == torch.bfloat16 else 1)
    L = _lib.load("tuned")
    fn = L.apc_skinny_gemm_bf16 if M <= SKINNY_MAX_ROWS else L.apc_gemm_bf16
    _lib.check(fn(a.data_ptr(), lda, w.data_ptr(), ldw, out.data_ptr(), ldc, M, N, K, mode, _ops._stream()),
               "gemm_bf16")


def swiglu_bf16(h: torch.Tensor, w_gate_up: torch.Tensor, out: torch.Tensor) -> None:
    """out[t, f] = silu(h . Wg[f]) * (h . Wu[f]), w_gate_up = [Wg; Wu] ([2F, K])."""
    _ops._gpu(h, w_gate_up, out)
    M, K = h.shape
    F = out.shape[1]
    _ops._need(w_gate_up.shape == (2 * F, K) and w_gate_up.is_contiguous(), "swiglu: weights must be [2F, K]")
    _ops._need(out.shape[0] == M, "swiglu: out rows differ from h rows")
    if not _mfma_ok(h, w_gate_up) or out.dtype != torch.bfloat16:
        gu = torch.empty((M, 2 * F), dtype=out.dtype, device=h.device)
        _ops.gemm_plain(h, w_gate_up, gu)
        return _ops.silu_mul(gu, out)
    lda, ldc = _ops._rows(h, "h"), _ops._rows(out, "out")
    wg, wu = w_gate_up[:F], w_gate_up[F:]
    L = _lib.load("tuned")
    fn = L.apc_skinny_swiglu_bf16 if M <= SKINNY_MAX_ROWS else L.apc_gemm_swiglu_bf16
    _lib.check(fn(h.data_ptr(), lda, wg.data_ptr(), wu.data_ptr(), K, out.data_ptr(), ldc, M, F, K, _ops._stream()),
               "swiglu_bf16")


def _keys_per_part(n_rows: int, n_kv_heads: int, max_context: int) -> int:
    """Keys one wave covers in the decode kernel: as many as leave about 2,000 waves on the chip."""
    kw = 32
    while kw < 1024 and n_rows * n_kv_heads * (-(-max_context // (kw * 2))) >= 2048:
        kw *= 2
    return kw


def attention_bf16(q: torch.Tensor, q_off: int, out: torch.Tensor, n_heads: int, n_kv_heads: int, head_dim: int,
                   cache: torch.Tensor, page_tokens: int, block_table: torch.Tensor, step, window: int = 0,
                   scale: Optional[float] = None) -> bool:
    """Attention of a whole step: single-row segments on the split-key decode kernel, longer segments on the
    tiled prefill kernel.  Returns False (nothing done) if the sizes are not ones these kernels take."""
    _ops._gpu(q, out, cache, block_table)
    ldq, ldo = _ops._rows(q, "attention q"), _ops._rows(out, "attention out")
    T = q.shape[0]
    if (head_dim % 16 or head_dim > 256 or page_tokens % 8 or ldq % 8 or q_off % 8 or not _aligned(q, cache)
            or q.dtype != torch.bfloat16 or cache.dtype != torch.bfloat16 or out.dtype != torch.bfloat16):
        return False
    _ops._need(q_off + n_heads * head_dim <= q.shape[1], "attention: q heads exceed the row")
    _ops._need(out.shape == (T, n_heads * head_dim), "attention out must be [rows, heads*head_dim]")
    _ops._need(n_heads % n_kv_heads == 0, "heads must be a multiple of kv heads")
    _ops._need(cache.dim() == 5 and cache.is_contiguous()
               and tuple(cache.shape[1:]) == (2, n_kv_heads, page_tokens, head_dim),
               f"cache must be [pages, 2, {n_kv_heads}, {page_tokens}, {head_dim}], got {tuple(cache.shape)}")
    _ops._need(block_table.dim() == 2 and block_table.dtype == torch.int32 and block_table.is_contiguous(),
               "block table must be contiguous int32 [segments, blocks]")
    _ops._need(step.positions.numel() >= T and step.row_seg.numel() >= T, "step rows differ from q rows")
    sc = (1.0 / math.sqrt(head_dim)) if scale is None else float(scale)
    L = _lib.load("tuned")
    stream = _ops._stream()
    if step.n_tiles:
        _lib.check(L.apc_attention_prefill_bf16(
            q.data_ptr(), ldq, q_off, out.data_ptr(), ldo, n_heads, n_kv_heads, head_dim, cache.data_ptr(),
            page_tokens, block_table.data_ptr(), block_table.shape[1], step.positions.data_ptr(),
            step.row_seg.data_ptr(), step.tile_row0.data_ptr(), step.tile_rows.data_ptr(), step.n_tiles,
            int(window), sc, stream), "attention_prefill_bf16")
    if step.n_decode_rows:
        n = step.n_decode_rows
        span = min(step.max_decode_context, window) if window else step.max_decode_context
        kw = _keys_per_part(n, n_kv_heads, span)
        n_parts = -(-step.max_decode_context // kw)
        ws = torch.empty(n * n_heads * n_parts * (head_dim + 2), dtype=torch.float32, device=q.device)
        rows = step.decode_rows.data_ptr() if step.decode_rows is not None else 0
        _lib.check(L.apc_attention_decode_bf16(
            q.data_ptr(), ldq, q_off, out.data_ptr(), ldo, n, n_heads, n_kv_heads, head_dim, cache.data_ptr(),
            page_tokens, block_table.data_ptr(), block_table.shape[1], step.positions.data_ptr(),
            step.row_seg.data_ptr(), rows, int(window), sc, kw, n_parts, ws.data_ptr(), stream),
            "attention_decode_bf16")
    return True
