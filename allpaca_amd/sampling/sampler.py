"""Chooses tokens from logits on the GPU.

Greedy rows (temperature <= 1e-5) take the first maximum; the others are sampled
by temperature / top-k / top-p with a uniform number that depends on (seed,
index of the generated token) only, so a request draws the same tokens alone,
in any batch, and after it was preempted and recomputed.  The reference keeps a
sequential generator per request (crates/allpaca-core/src/sampling.rs:5-8,
55-67), which ties a draw to how often the generator was used before."""
from __future__ import annotations

from typing import List, Sequence

import numpy as np
import torch

from ..kernels import ops
from .params import GenerationParams

_M64 = (1 << 64) - 1


def _splitmix64(x: int) -> int:
    x = (x + 0x9E3779B97F4A7C15) & _M64
    z = x
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M64
    return z ^ (z >> 31)


def uniform_for(seed: int, index: int) -> float:
    """A float32 in [0, 1) for the `index`-th generated token of a request with `seed`."""
    h = _splitmix64(_splitmix64(seed & _M64) ^ ((index + 1) * 0xD6E8FEB86659FD93 & _M64))
    return float(np.float32((h >> 40) / float(1 << 24)))


def _splitmix64_many(x: np.ndarray) -> np.ndarray:
    """`_splitmix64` of every element of a uint64 array (the arithmetic wraps modulo 2^64, as masked Python ints do)."""
    x = x + np.uint64(0x9E3779B97F4A7C15)
    z = (x ^ (x >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
    z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
    return z ^ (z >> np.uint64(31))


def uniforms_for(seeds: Sequence[int], indices: Sequence[int]) -> np.ndarray:
    """`uniform_for` of every (seed, index) pair, as a float32 array."""
    sd = np.asarray([s & _M64 for s in seeds], dtype=np.uint64)
    ix = (np.asarray(indices, dtype=np.uint64) + np.uint64(1)) * np.uint64(0xD6E8FEB86659FD93)
    h = _splitmix64_many(_splitmix64_many(sd) ^ ix)
    return ((h >> np.uint64(40)).astype(np.float64) / float(1 << 24)).astype(np.float32)


class Sampler:
    def __init__(self, device: torch.device, default_seed: int):
        self.device = device
        self.default_seed = default_seed
        self._pinned = [None, None]   # token ids come back through pinned memory; two results may be under way
        # the rows' parameters go the other way through pinned memory too (float32 [4, cap]: temperature, top-p, the
        # uniform number, top-k as bits), one buffer per result under way, so that a step queued behind a running one
        # does not wait for it in a copy from pageable memory
        self._params_host = [None, None]
        self._params_dev = [None, None]
        self._params_copied = [None, None]
        self._turn = 0

    def _upload(self, params: Sequence[GenerationParams], indices: Sequence[int]) -> torch.Tensor:
        """float32 [4, cap] on the device: rows temperature, top-p, uniform number, top-k (an int32 seen as float32)."""
        R, t = len(params), self._turn
        if self._params_host[t] is None or self._params_host[t].shape[1] < R:
            cap = max(64, 1 << (R - 1).bit_length())
            self._params_host[t] = torch.empty((4, cap), dtype=torch.float32).pin_memory()
            self._params_dev[t] = torch.empty((4, cap), dtype=torch.float32, device=self.device)
            self._params_copied[t] = None
        if self._params_copied[t] is not None:
            self._params_copied[t].synchronize()     # the copy out of this buffer two results ago
        host = self._params_host[t].numpy()
        host[0, :R] = [p.temperature for p in params]
        host[1, :R] = [p.top_p for p in params]
        host[2, :R] = uniforms_for([self.default_seed if p.seed is None else p.seed for p in params], indices)
        host[3, :R].view(np.int32)[:] = [p.top_k for p in params]
        self._params_dev[t].copy_(self._params_host[t], non_blocking=True)
        self._params_copied[t] = torch.cuda.Event()
        self._params_copied[t].record()
        return self._params_dev[t]

    def sample(self, logits: torch.Tensor, params: Sequence[GenerationParams], indices: Sequence[int]) -> List[int]:
        """logits: float32 [R, V] on the GPU; params[r] and indices[r] (how many tokens row r's request
        has generated so far) choose the rule and the random number of row r."""
        return self.launch(logits, params, indices).wait()

    def launch(self, logits: torch.Tensor, params: Sequence[GenerationParams], indices: Sequence[int]) -> "Pending":
        """The same without waiting: the kernels and the copy of the token ids to the host are queued; `wait()` of
        the result gives the ids.  The caller may do other work on the host in between."""
        R = logits.shape[0]
        out = torch.empty(R, dtype=torch.int32, device=self.device)
        self._turn ^= 1
        if all(p.greedy for p in params):
            ops.argmax_rows(logits, out)
        else:
            f = self._upload(params, indices)
            ops.sample_rows(logits, f[0, :R], f[3, :R].view(torch.int32), f[1, :R], f[2, :R], out,
                            any_top_k=any(p.top_k > 0 for p in params),
                            any_top_p=any(0.0 <= p.top_p < 1.0 for p in params),
                            few_after_top_k=all(p.greedy or 0 < p.top_k <= 1024 for p in params))
        if self._pinned[self._turn] is None or self._pinned[self._turn].numel() < R:
            self._pinned[self._turn] = torch.empty(max(R, 64), dtype=torch.int32).pin_memory()
        pinned = self._pinned[self._turn]
        pinned[:R].copy_(out, non_blocking=True)
        done = torch.cuda.Event()
        done.record()
        return Pending(pinned, R, done, out)


class Pending:
    """Token ids on their way to the host; `device` holds them on the GPU (int32 [n])."""

    def __init__(self, pinned: torch.Tensor, n: int, done: torch.cuda.Event, device: torch.Tensor):
        self.pinned, self.n, self.done, self.device = pinned, n, done, device

    def wait(self) -> List[int]:
        self.done.synchronize()
        return self.pinned[:self.n].tolist()
