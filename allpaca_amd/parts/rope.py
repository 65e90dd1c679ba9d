"""Rotary position encoding, NeoX pairing (i, i + rot/2), with optional
Llama-3 frequency scaling.

inv_freq[i] = theta^(-2i/rot) (the reference's stream theta_scale^i with
theta_scale = theta^(-2/n_rot), crates/allpaca-cpu/src/kernels.rs:640-683; the
HF safetensors path uses this pairing, crates/allpaca-core/src/model.rs:7937).
The reference has no frequency scaling on its llama path
(crates/allpaca-core/src/model.rs:181-274); the "llama3" rule is the published
one: by wavelength 2*pi/inv_freq, short waves keep their frequency, long waves
are slowed by `factor`, and the band between is blended linearly.

Angles are formed in 64-bit on the host (position * inv_freq) and the cosines
and sines rounded once to float32: a table [positions, 2, rot/2]."""
from __future__ import annotations

import math
from typing import Mapping, Optional

import numpy as np
import torch

from ..kernels import ops
from .base import POSITION_ENCODINGS, PositionEncoding, Runtime


def inverse_frequencies(rot: int, theta: float, scaling: Optional[Mapping] = None) -> np.ndarray:
    i = np.arange(rot // 2, dtype=np.float64)
    inv = np.power(float(theta), -2.0 * i / rot)
    if not scaling:
        return inv
    kind = scaling.get("rope_type", "llama3")
    if kind != "llama3":
        raise ValueError(f"rope scaling {kind!r} is not supported (known: 'llama3')")
    factor = float(scaling["factor"])
    lo, hi = float(scaling["low_freq_factor"]), float(scaling["high_freq_factor"])
    orig = float(scaling["original_max_position_embeddings"])
    wavelen = 2.0 * math.pi / inv
    smooth = (orig / wavelen - lo) / (hi - lo)
    blended = (1.0 - smooth) * inv / factor + smooth * inv
    return np.where(wavelen < orig / hi, inv, np.where(wavelen > orig / lo, inv / factor, blended))


@POSITION_ENCODINGS.register("rope")
class RotaryEncoding(PositionEncoding):
    graph_safe = True

    def __init__(self, head_dim: int, theta: float, rotary_dim: Optional[int] = None,
                 scaling: Optional[Mapping] = None):
        self.head_dim = int(head_dim)
        self.rot = int(rotary_dim) if rotary_dim else self.head_dim
        if self.rot % 2 or self.rot > self.head_dim:
            raise ValueError(f"rotary width {self.rot} must be even and at most head_dim {self.head_dim}")
        self.theta = float(theta)
        self.scaling = dict(scaling) if scaling else None
        self.inv_freq = inverse_frequencies(self.rot, self.theta, self.scaling)

    def bind(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        pos = np.arange(rt.max_positions, dtype=np.float64)[:, None]
        ang = pos * self.inv_freq[None, :]
        table = np.stack([np.cos(ang), np.sin(ang)], axis=1).astype(np.float32)  # [positions, 2, rot/2]
        self.cos_sin = torch.from_numpy(table).to(rt.device).contiguous()

    def fused(self):
        return self.rot, self.cos_sin

    def apply(self, qkv, q_off, k_off, n_heads, n_kv_heads, head_dim, positions) -> None:
        ops.rope_kv_write(qkv, q_off, k_off, 0, n_heads, n_kv_heads, head_dim, self.rot, self.cos_sin, positions)


@POSITION_ENCODINGS.register("none")
class NoEncoding(PositionEncoding):
    graph_safe = True

    def __init__(self, **_):
        pass

    def fused(self):
        return 0, None

    def apply(self, *a, **k) -> None:
        return None
