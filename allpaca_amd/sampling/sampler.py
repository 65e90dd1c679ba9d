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


class Sampler:
    def __init__(self, device: torch.device, default_seed: int):
        self.device = device
        self.default_seed = default_seed
        self._pinned = [None, None]   # token ids come back through pinned memory; two results may be under way
        self._turn = 0

    def sample(self, logits: torch.Tensor, params: Sequence[GenerationParams], indices: Sequence[int]) -> List[int]:
        """logits: float32 [R, V] on the GPU; params[r] and indices[r] (how many tokens row r's request
        has generated so far) choose the rule and the random number of row r."""
        return self.launch(logits, params, indices).wait()

    def launch(self, logits: torch.Tensor, params: Sequence[GenerationParams], indices: Sequence[int]) -> "Pending":
        """The same without waiting: the kernels and the copy of the token ids to the host are queued; `wait()` of
        the result gives the ids.  The caller may do other work on the host in between."""
        R = logits.shape[0]
        out = torch.empty(R, dtype=torch.int32, device=self.device)
        if all(p.greedy for p in params):
            ops.argmax_rows(logits, out)
        else:
            host = np.empty((4, R), dtype=np.float32)
            ks = np.empty(R, dtype=np.int32)
            for r, (p, i) in enumerate(zip(params, indices)):
                host[0, r] = p.temperature
                host[1, r] = p.top_p
                host[2, r] = uniform_for(self.default_seed if p.seed is None else p.seed, i)
                ks[r] = p.top_k
            f = torch.from_numpy(host).to(self.device)
            k = torch.from_numpy(ks).to(self.device)
            ops.sample_rows(logits, f[0], k, f[1], f[2], out)
        self._turn ^= 1
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
