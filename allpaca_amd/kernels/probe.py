"""Measured peaks of the card this process runs on: what a streaming read and a loop of MFMAs reach, so that a
kernel's share of the published peak can be split into "the kernel" and "the hardware"."""
from __future__ import annotations

import torch

from . import lib as _lib
from . import ops as _ops


def read_bandwidth(gib: float = 8.0, blocks: int = 256 * 8, unroll: int = 8, repeats: int = 3, once: bool = True) -> float:
    """GB/s of reading `gib` GiB of device memory once with 16-byte loads (best of `repeats`); `once`: with loads that
    the caches do not keep, as the decode kernels read weights, keys and values."""
    L = _lib.load("bench")
    n = int(gib * 2 ** 30) // 16 * 16
    buf = torch.empty(n, dtype=torch.uint8, device="cuda")
    buf.fill_(1)
    out = torch.empty(blocks, dtype=torch.float32, device="cuda")
    best = 0.0
    for _ in range(repeats + 1):
        t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0.record()
        _lib.check(L.apc_probe_read(buf.data_ptr(), n, out.data_ptr(), blocks, unroll, int(once), _ops._stream()), "probe_read")
        t1.record()
        t1.synchronize()
        best = max(best, n / (t0.elapsed_time(t1) * 1e-3) / 1e9)
    del buf
    torch.cuda.empty_cache()
    return best


def mfma_rate(iters: int = 20000, blocks: int = 256 * 4, repeats: int = 2) -> float:
    """TFLOP/s of independent v_mfma_f32_32x32x16_bf16 from registers on every compute unit."""
    L = _lib.load("bench")
    out = torch.empty(blocks * 256, dtype=torch.float32, device="cuda")
    best = 0.0
    for _ in range(repeats + 1):
        t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0.record()
        _lib.check(L.apc_probe_mfma(iters, out.data_ptr(), blocks, _ops._stream()), "probe_mfma")
        t1.record()
        t1.synchronize()
        flops = blocks * 4 * iters * 8 * 2 * 32 * 32 * 16
        best = max(best, flops / (t0.elapsed_time(t1) * 1e-3) / 1e12)
    return best
