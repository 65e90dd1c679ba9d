"""Checked wrappers around the HIP entry points.  Each takes torch tensors that
live on the GPU, checks on the host that shapes, strides and element types are
what the kernel and its grid assume, and launches on torch's current stream.
Nothing here computes on the CPU and nothing falls back to a library."""
from __future__ import annotations

import math
import os
from typing import Optional

import torch

from . import lib as _lib
from .packing import PackedWeight

F32, BF16, I32 = 0, 1, 2
_CODES = {torch.float32: F32, torch.bfloat16: BF16, torch.int32: I32}


def _code(t: torch.Tensor) -> int:
    try:
        return _CODES[t.dtype]
    except KeyError:
        raise TypeError(f"element type {t.dtype} is not handled by the kernels (float32, bfloat16, int32)") from None


def _stream() -> int:
    """The current HIP stream's handle (the raw call: `torch.cuda.current_stream()` builds an object each time)."""
    return torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice())


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise ValueError(msg)


def _gpu(*ts: Optional[torch.Tensor]) -> None:
    for t in ts:
        if t is not None and not t.is_cuda:
            raise ValueError("kernel operands must live on the GPU (there is no CPU path)")


def _rows(t: torch.Tensor, what: str) -> int:
    """A [rows, cols] view with unit column stride; returns its row stride."""
    if not (t.dim() == 2):
        raise ValueError(f"{what}: expected 2 dimensions, got shape {tuple(t.shape)}")
    if not (t.shape[1] == 0 or t.stride(1) == 1):
        raise ValueError(f"{what}: columns must be contiguous")
    return t.stride(0) if t.shape[0] > 1 else max(t.stride(0), t.shape[1])


def _i32(t: Optional[torch.Tensor], n: int, what: str) -> int:
    if t is None:
        return 0
    if not (t.dtype == torch.int32 and t.is_contiguous() and t.numel() >= n):
        raise ValueError(f"{what}: need >= {n} contiguous int32")
    return t.data_ptr()


# --------------------------------------------------------------------------- plain library
def embed_rows(table, tokens: torch.Tensor, out: torch.Tensor) -> None:
    """out[t] = table[tokens[t]]; the table is a [vocab, dim] matrix or its tiled form (`PackedWeight`)."""
    T = tokens.numel()
    ldo = _rows(out, "embed out")
    if isinstance(table, PackedWeight):
        _gpu(table.data, tokens, out)
        _need(out.shape == (T, table.K), "embed out must be [tokens, dim]")
        L = _lib.load("plain")
        _lib.check(L.apc_embed_rows_tiled(table.data.data_ptr(), table.chunks, _i32(tokens, T, "tokens"),
                                          out.data_ptr(), _code(out), T, table.K, ldo, _stream()), "embed_rows_tiled")
        return
    _gpu(table, tokens, out)
    _need(table.dim() == 2 and table.is_contiguous(), "embedding table must be a contiguous [vocab, dim] matrix")
    _need(out.shape[0] == T and out.shape[1] == table.shape[1], "embed out must be [tokens, dim]")
    L = _lib.load("plain")
    _lib.check(L.apc_embed_rows(table.data_ptr(), _code(table), _i32(tokens, T, "tokens"), out.data_ptr(), _code(out),
                                T, table.shape[1], ldo, _stream()), "embed_rows")


def gather_rows(x: torch.Tensor, rows: torch.Tensor, out: torch.Tensor) -> None:
    _gpu(x, rows, out)
    R = rows.numel()
    ldx, ldo = _rows(x, "gather x"), _rows(out, "gather out")
    _need(out.shape == (R, x.shape[1]) and out.dtype == x.dtype, "gather out must be [rows, dim] of x's type")
    L = _lib.load("plain")
    _lib.check(L.apc_gather_rows(x.data_ptr(), _code(x), ldx, _i32(rows, R, "rows"), out.data_ptr(), ldo, R, x.shape[1],
                                 _stream()), "gather_rows")


def rmsnorm_rows(x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor,
                 rows: Optional[torch.Tensor] = None) -> None:
    _gpu(x, weight, out, rows)
    ldx, ldo = _rows(x, "rmsnorm x"), _rows(out, "rmsnorm out")
    R = out.shape[0]
    D = x.shape[1]
    if not (weight.dtype == torch.float32 and weight.is_contiguous() and weight.numel() == D):
        raise ValueError(f"rmsnorm weight must be float32 [{D}]")
    _need(out.shape[1] == D, "rmsnorm out width differs from x")
    _need(rows is not None or x.shape[0] == R, "rmsnorm: out rows differ from x rows")
    L = _lib.load("plain")
    _lib.check(L.apc_rmsnorm_rows(x.data_ptr(), _code(x), ldx, _i32(rows, R, "rows"), weight.data_ptr(), float(eps),
                                  out.data_ptr(), _code(out), ldo, R, D, _stream()), "rmsnorm_rows")


def add_into(acc: torch.Tensor, y: torch.Tensor) -> None:
    _gpu(acc, y)
    lda, ldy = _rows(acc, "add acc"), _rows(y, "add y")
    _need(acc.dtype == torch.float32, "the residual sum is kept in float32")
    _need(acc.shape == y.shape, "add_into: shapes differ")
    L = _lib.load("plain")
    _lib.check(L.apc_add_into(acc.data_ptr(), lda, y.data_ptr(), _code(y), ldy, acc.shape[0], acc.shape[1], _stream()),
               "add_into")


def silu_mul(gate_up: torch.Tensor, out: torch.Tensor) -> None:
    _gpu(gate_up, out)
    ldg, ldo = _rows(gate_up, "silu_mul in"), _rows(out, "silu_mul out")
    T, F = out.shape
    _need(gate_up.shape == (T, 2 * F), "silu_mul: input must be [rows, 2*F] (gate columns, then up columns)")
    L = _lib.load("plain")
    for r0 in range(0, T, 32768):
        n = min(32768, T - r0)
        _lib.check(L.apc_silu_mul(gate_up[r0:].data_ptr(), _code(gate_up), ldg, out[r0:].data_ptr(), _code(out), ldo,
                                  n, F, _stream()), "silu_mul")


def cast(src: torch.Tensor, dst: torch.Tensor) -> None:
    _gpu(src, dst)
    _need(src.is_contiguous() and dst.is_contiguous() and src.numel() == dst.numel(), "cast: contiguous, same count")
    L = _lib.load("plain")
    _lib.check(L.apc_cast(src.data_ptr(), _code(src), dst.data_ptr(), _code(dst), src.numel(), _stream()), "cast")


def rope_kv_write(qkv: torch.Tensor, q_off: int, k_off: int, v_off: int, n_heads: int, n_kv_heads: int, head_dim: int,
                  rot: int, cos_sin: Optional[torch.Tensor], positions: torch.Tensor,
                  row_seg: Optional[torch.Tensor] = None, block_table: Optional[torch.Tensor] = None,
                  cache: Optional[torch.Tensor] = None, page_tokens: int = 0) -> None:
    """Rotate q (and k) of every row by its position; with `cache`, write rotated k and v into the pages."""
    _gpu(qkv, cos_sin, positions, row_seg, block_table, cache)
    ld = _rows(qkv, "qkv")
    T = qkv.shape[0]
    width = qkv.shape[1]
    _need(q_off + n_heads * head_dim <= width and k_off + n_kv_heads * head_dim <= width
          and v_off + n_kv_heads * head_dim <= width, "qkv: head ranges exceed the row")
    _need(rot % 2 == 0 and 0 <= rot <= head_dim, "rotated width must be even and at most head_dim")
    if rot:
        _need(cos_sin is not None and cos_sin.dtype == torch.float32 and cos_sin.is_contiguous()
              and cos_sin.dim() == 3 and cos_sin.shape[1] == 2 and cos_sin.shape[2] == rot // 2,
              "cos/sin table must be float32 [positions, 2, rot/2]")
    max_blocks = 0
    if cache is not None:
        _need(block_table is not None and row_seg is not None, "cache write needs a block table and row segments")
        if not (cache.dim() == 5 and cache.is_contiguous()
                and tuple(cache.shape[1:]) == (2, n_kv_heads, page_tokens, head_dim)):
            raise ValueError(f"cache must be [pages, 2, {n_kv_heads}, {page_tokens}, {head_dim}], "
                             f"got {tuple(cache.shape)}")
        _need(block_table.dim() == 2 and block_table.dtype == torch.int32 and block_table.is_contiguous(),
              "block table must be contiguous int32 [segments, blocks]")
        max_blocks = block_table.shape[1]
    if (not FORCE_PLAIN and qkv.dtype == torch.bfloat16 and (cache is None or cache.dtype == torch.bfloat16)
            and head_dim % 8 == 0 and rot % 16 == 0 and ld % 8 == 0 and q_off % 8 == 0 and k_off % 8 == 0
            and v_off % 8 == 0 and qkv.data_ptr() % 16 == 0):
        # the same operation 16 bytes a lane (library `tuned`)
        _lib.check(_lib.load("tuned").apc_rope_kv_write_bf16(
            qkv.data_ptr(), ld, q_off, k_off, v_off, T, n_heads, n_kv_heads, head_dim, rot,
            cos_sin.data_ptr() if rot else 0, _i32(positions, T, "positions"),
            _i32(row_seg, T, "row_seg") if row_seg is not None else 0,
            block_table.data_ptr() if block_table is not None else 0, max_blocks,
            cache.data_ptr() if cache is not None else 0, page_tokens, _stream()), "rope_kv_write_bf16")
        return
    L = _lib.load("plain")
    _lib.check(L.apc_rope_kv_write(
        qkv.data_ptr(), _code(qkv), ld, q_off, k_off, v_off, T, n_heads, n_kv_heads, head_dim, rot,
        cos_sin.data_ptr() if rot else 0, _i32(positions, T, "positions"),
        _i32(row_seg, T, "row_seg") if row_seg is not None else 0,
        block_table.data_ptr() if block_table is not None else 0, max_blocks,
        cache.data_ptr() if cache is not None else 0, _code(cache) if cache is not None else 0, page_tokens,
        _stream()), "rope_kv_write")


def gemm_plain(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, accumulate: bool = False) -> None:
    """out = a . w^T, or out += a . w^T (out float32), in true 32-bit arithmetic."""
    _gpu(a, w, out)
    lda, ldw, ldc = _rows(a, "gemm a"), _rows(w, "gemm w"), _rows(out, "gemm out")
    M, K = a.shape
    N = w.shape[0]
    if not (w.shape[1] == K):
        raise ValueError(f"gemm: a is [*, {K}] but w is {tuple(w.shape)}")
    if not (out.shape == (M, N)):
        raise ValueError(f"gemm: out must be [{M}, {N}], got {tuple(out.shape)}")
    _need(not accumulate or out.dtype == torch.float32, "gemm: accumulation needs a float32 destination")
    L = _lib.load("plain")
    for r0 in range(0, M, 1 << 21):  # grid.y limit: 65535 tiles of 64 rows
        n = min(1 << 21, M - r0)
        _lib.check(L.apc_gemm_plain(a[r0:].data_ptr(), _code(a), lda, w.data_ptr(), _code(w), ldw,
                                    out[r0:].data_ptr(), _code(out), ldc, n, N, K, 1 if accumulate else 0, _stream()),
                   "gemm_plain")


def paged_attention_plain(q: torch.Tensor, q_off: int, out: torch.Tensor, n_heads: int, n_kv_heads: int,
                          head_dim: int, cache: torch.Tensor, page_tokens: int, block_table: torch.Tensor,
                          positions: torch.Tensor, row_seg: torch.Tensor, window: int = 0,
                          scale: Optional[float] = None) -> None:
    _gpu(q, out, cache, block_table, positions, row_seg)
    ldq, ldo = _rows(q, "attention q"), _rows(out, "attention out")
    T = q.shape[0]
    _need(q_off + n_heads * head_dim <= q.shape[1], "attention: q heads exceed the row")
    _need(out.shape == (T, n_heads * head_dim), "attention out must be [rows, heads*head_dim]")
    _need(n_heads % n_kv_heads == 0, "heads must be a multiple of kv heads")
    _need(head_dim <= 256, "plain attention handles head_dim <= 256")
    if not (cache.dim() == 5 and cache.is_contiguous()
            and tuple(cache.shape[1:]) == (2, n_kv_heads, page_tokens, head_dim)):
        raise ValueError(f"cache must be [pages, 2, {n_kv_heads}, {page_tokens}, {head_dim}], got {tuple(cache.shape)}")
    _need(block_table.dim() == 2 and block_table.dtype == torch.int32 and block_table.is_contiguous(),
          "block table must be contiguous int32 [segments, blocks]")
    L = _lib.load("plain")
    sc = (1.0 / math.sqrt(head_dim)) if scale is None else float(scale)
    _lib.check(L.apc_paged_attention_plain(
        q.data_ptr(), _code(q), ldq, q_off, out.data_ptr(), _code(out), ldo, T, n_heads, n_kv_heads, head_dim,
        cache.data_ptr(), _code(cache), page_tokens, block_table.data_ptr(), block_table.shape[1],
        _i32(positions, T, "positions"), _i32(row_seg, T, "row_seg"), int(window), sc, _stream()),
        "paged_attention_plain")


def argmax_rows(logits: torch.Tensor, out: torch.Tensor) -> None:
    _gpu(logits, out)
    ld = _rows(logits, "logits")
    R, V = logits.shape
    _need(logits.dtype == torch.float32, "logits are float32")
    L = _lib.load("plain")
    scratch = torch.empty(2 * R * 64, dtype=torch.int32, device=logits.device) if V >= 8192 else None
    _lib.check(L.apc_argmax_rows(logits.data_ptr(), ld, R, V, _i32(out, R, "argmax out"),
                                 scratch.data_ptr() if scratch is not None else 0, _stream()), "argmax_rows")


def sample_rows(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
                uniform: torch.Tensor, out: torch.Tensor, any_top_k: bool = True, any_top_p: bool = True,
                few_after_top_k: bool = False, one_block: bool = False) -> None:
    """One token a row by temperature / top-k / top-p with the row's uniform number.  `any_top_k`, `any_top_p`: whether
    some row may ask for that cut; `few_after_top_k`: every row that samples has 0 < top-k <= 1,024.  A caller that
    knows its rows saves the launches that none of them needs; a row for which its word is wrong still gets its
    token, slowly.  `one_block`: the kernel without working memory, one block a row."""
    _gpu(logits, temperature, top_k, top_p, uniform, out)
    ld = _rows(logits, "logits")
    R, V = logits.shape
    _need(logits.dtype == torch.float32, "logits are float32")
    for t, name in ((temperature, "temperature"), (top_p, "top_p"), (uniform, "uniform")):
        if not (t.dtype == torch.float32 and t.is_contiguous() and t.numel() >= R):
            raise ValueError(f"{name}: float32 [{R}]")
    L = _lib.load("plain")
    kib = 0 if one_block else L.apc_sample_rows_scratch_kib(R)
    scratch = torch.empty(kib * 1024, dtype=torch.uint8, device=logits.device) if kib else None
    _lib.check(L.apc_sample_rows(logits.data_ptr(), ld, R, V, temperature.data_ptr(), _i32(top_k, R, "top_k"),
                                 top_p.data_ptr(), uniform.data_ptr(), _i32(out, R, "sample out"),
                                 scratch.data_ptr() if scratch is not None else 0, kib * 1024,
                                 (1 if any_top_k else 0) | (2 if any_top_p else 0) | (4 if few_after_top_k else 0),
                                 _stream()),
               "sample_rows")


# --------------------------------------------------------------------------- dispatch
# With FORCE_PLAIN every step runs on the plain kernels whatever the element type
# (used by tests to check one tuned kernel at a time against the same model).
FORCE_PLAIN = os.environ.get("ALLPACA_AMD_PLAIN", "0") == "1"


def _tuned_ok(*ts: torch.Tensor) -> bool:
    return (not FORCE_PLAIN) and all(t.dtype == torch.bfloat16 for t in ts)


def prepare_matrix(w: torch.Tensor, run_dtype: torch.dtype):
    """How a weight matrix [out, in] is kept on the GPU: a bfloat16 matrix of a bfloat16 run in the tiled layout
    of the MFMA kernels (if its width is a multiple of 8), anything else as it is."""
    from .packing import can_pack, pack_mfma
    if run_dtype == torch.bfloat16 and not FORCE_PLAIN and w.is_cuda and can_pack(w):
        return pack_mfma(w)
    return w.contiguous()


def linear(a: torch.Tensor, w, out: torch.Tensor, accumulate: bool = False, emit=None) -> None:
    """out = a . w^T (or out += ..., out float32).  A tiled bfloat16 weight runs on the MFMA kernels.
    `emit` (with accumulate): an object with `weight` (an RMS norm's) whose `raw` and `ss` are filled with what
    that norm's next product needs, where there is a kernel for these sizes; else it is left as it is."""
    if isinstance(w, PackedWeight):
        from . import tuned
        if emit is not None and accumulate:
            left = tuned.gemm_emit_bf16(a, w, out, emit.weight)
            if left is not None:
                emit.raw, emit.ss = left
                return
        tuned.gemm_bf16(a, w, out, accumulate)
    else:
        gemm_plain(a, w, out, accumulate)


def swiglu(h: torch.Tensor, w_gate_up, out: torch.Tensor) -> None:
    """out[t, f] = silu(h . Wg[f]) * (h . Wu[f]); w_gate_up is [Wg; Wu] of shape [2F, D], or the pair of
    their tiled forms."""
    if isinstance(w_gate_up, tuple):
        from . import tuned
        tuned.swiglu_bf16(h, w_gate_up[0], w_gate_up[1], out)
        return
    T, F = out.shape
    gu = torch.empty((T, 2 * F), dtype=torch.float32 if h.dtype == torch.float32 else out.dtype, device=h.device)
    gemm_plain(h, w_gate_up, gu)
    silu_mul(gu, out)


def linear_pre(raw: torch.Tensor, ss: torch.Tensor, eps: float, w, out: torch.Tensor) -> bool:
    """The product of a normalised row from what `linear(..., emit=...)` left; False if there is no kernel for
    these sizes (nothing is done then)."""
    if isinstance(w, PackedWeight) and not FORCE_PLAIN:
        from . import tuned
        return tuned.gemm_pre_bf16(raw, ss, eps, w, out)
    return False


def qkv_rope_write(a: torch.Tensor, pre, w, q_out: torch.Tensor, n_heads: int, n_kv_heads: int, head_dim: int,
                   cos_sin: torch.Tensor, positions: torch.Tensor, row_seg: torch.Tensor, block_table: torch.Tensor,
                   cache: torch.Tensor, page_tokens: int) -> bool:
    """The product for q, k and v, the rotation of whole q and k heads and the write of k and v into the pages in
    one kernel (few rows; `pre` = (ss, eps) if `a` is a row that `linear(..., emit=...)` left, else None).  False if
    there is no such kernel for these sizes (nothing is done then)."""
    if isinstance(w, PackedWeight) and not FORCE_PLAIN:
        from . import tuned
        return tuned.qkv_rope_bf16(a, pre, w, q_out, n_heads, n_kv_heads, head_dim, cos_sin, positions, row_seg,
                                   block_table, cache, page_tokens)
    return False


def swiglu_pre(raw: torch.Tensor, ss: torch.Tensor, eps: float, w_gate_up, out: torch.Tensor) -> bool:
    if isinstance(w_gate_up, tuple) and not FORCE_PLAIN:
        from . import tuned
        return tuned.swiglu_pre_bf16(raw, ss, eps, w_gate_up[0], w_gate_up[1], out)
    return False


def attention_tile_rows(run_dtype: torch.dtype = torch.bfloat16) -> int:
    """Rows of a tile of the attention kernel that takes segments of several rows: the step packer cuts segments into
    such tiles (`StepInfo.tile_row0`, `tile_rows`).  The kernel's library says how many; the plain kernel, which
    32-bit runs use, does not look at tiles."""
    if run_dtype != torch.bfloat16 or FORCE_PLAIN:
        return 64
    return int(_lib.load("tuned").apc_attention_prefill_tile_rows())


def paged_attention(q: torch.Tensor, q_off: int, out: torch.Tensor, n_heads: int, n_kv_heads: int, head_dim: int,
                    cache: torch.Tensor, page_tokens: int, block_table: torch.Tensor, step, window: int = 0,
                    scale: Optional[float] = None) -> None:
    if _tuned_ok(q, cache, out):
        from . import tuned
        if tuned.attention_bf16(q, q_off, out, n_heads, n_kv_heads, head_dim, cache, page_tokens, block_table, step,
                                window, scale):
            return
    paged_attention_plain(q, q_off, out, n_heads, n_kv_heads, head_dim, cache, page_tokens, block_table,
                          step.positions, step.row_seg, window, scale)
