"""Shared by the tests: two tiny llama configurations that differ in every size
and option, model folders with random (or planted) weights in a temporary
place, the oracle's logits, and the ways a request's tokens are cut into steps."""
from __future__ import annotations

import functools
import math
import os
import shutil
import tempfile
from typing import Dict, List, Sequence

import numpy as np
import torch

import plain_llama as P

# Tiny A: MHA, head_dim 16, tied head, no scaling, sizes that are no power of two (176, 3 layers' worth below in B)
TINY_A = dict(
    architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=256, hidden_size=64, num_hidden_layers=2,
    num_attention_heads=4, num_key_value_heads=4, head_dim=16, intermediate_size=176, rms_norm_eps=1e-5,
    rope_theta=10000.0, rope_scaling=None, tie_word_embeddings=True, max_position_embeddings=128, hidden_act="silu")
# Tiny B: GQA 3:1, head_dim 32, untied head, llama3 scaling with all three regions, other eps/theta/vocab
TINY_B = dict(
    architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=1000, hidden_size=192, num_hidden_layers=3,
    num_attention_heads=6, num_key_value_heads=2, head_dim=32, intermediate_size=512, rms_norm_eps=1e-6,
    rope_theta=500000.0,
    rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=64),
    tie_word_embeddings=False, max_position_embeddings=256, hidden_act="silu")
# Tiny C: head_dim differs from hidden/heads, 5 heads over 1 kv head, odd widths, head_dim 48 (a multiple of 16 only)
TINY_C = dict(
    architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=515, hidden_size=120, num_hidden_layers=2,
    num_attention_heads=5, num_key_value_heads=1, head_dim=48, intermediate_size=200, rms_norm_eps=3e-6,
    rope_theta=250000.0,
    rope_scaling=dict(rope_type="llama3", factor=4.0, low_freq_factor=1.0, high_freq_factor=2.0,
                      original_max_position_embeddings=32),
    tie_word_embeddings=True, max_position_embeddings=320, hidden_act="silu")

CONFIGS = {"A": (TINY_A, 0, 0.0), "B": (TINY_B, 1, 0.1), "C": (TINY_C, 2, 0.05)}  # config, seed, norm_std

_TMP = None


def tmp_root() -> str:
    global _TMP
    if _TMP is None:
        _TMP = tempfile.mkdtemp(prefix="allpaca_amd_tests_")
        import atexit
        atexit.register(shutil.rmtree, _TMP, ignore_errors=True)
    return _TMP


@functools.lru_cache(maxsize=None)
def model_folder(name: str, dtype: str = "float32", sharp: bool = False) -> str:
    """A folder for tiny configuration `name`.  `sharp`: query and key projections
    scaled up so that attention is peaked (random N(0, 0.02) weights give scores of
    standard deviation ~0.05, almost uniform attention, which hides a wrong or missing
    key).  The scale is chosen for scores of standard deviation ~3, as in trained
    models: with unit-variance inputs a score is a sum of head_dim products of two
    N(0, s^2 0.02^2 D) numbers over sqrt(head_dim), of deviation s^2 0.02^2 D."""
    from allpaca_amd.weights import write_model_folder
    cfg, seed, norm_std = CONFIGS[name]
    path = os.path.join(tmp_root(), f"{name}_{dtype}_{'sharp' if sharp else 'plain'}")
    tdt = torch.float32 if dtype == "float32" else torch.bfloat16
    overrides = {}
    if sharp:
        from allpaca_amd.models import DecoderModel, describe_model
        from allpaca_amd.weights import random_tensors
        _, _, spec = describe_model(cfg)
        base = random_tensors(DecoderModel(spec).param_specs(), seed, torch.float32, 0.02, norm_std)
        for k, t in base.items():
            if k.endswith("q_proj.weight") or k.endswith("k_proj.weight"):
                overrides[k] = t * math.sqrt(3.0 / (0.02 ** 2 * cfg["hidden_size"]))
            if k.endswith("v_proj.weight") or k.endswith("o_proj.weight"):
                overrides[k] = t * 3.0
    write_model_folder(path, cfg, seed, tdt, std=0.02, norm_std=norm_std, overrides=overrides)
    return path


@functools.lru_cache(maxsize=None)
def oracle(folder: str):
    return P.read_model_folder(folder)


_ORACLE_CACHE: Dict = {}


def oracle_logits(folder: str, tokens: Sequence[int]) -> np.ndarray:
    key = (folder, tuple(tokens))
    if key not in _ORACLE_CACHE:
        cfg, w = oracle(folder)
        _ORACLE_CACHE[key] = P.llama_forward(cfg, w, list(tokens))
    return _ORACLE_CACHE[key]


def random_tokens(vocab: int, n: int, seed: int) -> List[int]:
    return np.random.default_rng(seed).integers(0, vocab, size=n).tolist()


def oracle_logits_bf16_storage(folder: str, tokens: Sequence[int]) -> np.ndarray:
    """The oracle with every stored activation rounded to bfloat16 and exact arithmetic otherwise."""
    key = (folder, tuple(tokens), "bf16")
    if key not in _ORACLE_CACHE:
        cfg, w = oracle(folder)
        _ORACLE_CACHE[key] = P.llama_forward(cfg, w, list(tokens), store=P.round_bf16)
    return _ORACLE_CACHE[key]


# ---- tolerances, fixed before any run ------------------------------------------
# float32 engine against the float64 oracle: absolute, on logits of magnitude ~0.3
F32_ATOL = 2e-5
# bfloat16 engine (bfloat16 weights, activations and cache; 32-bit sums) against the float64
# oracle on the same bfloat16 weights.  What bfloat16 storage of activations costs is not
# guessed: the oracle itself is run once more with its stored activations rounded to bfloat16
# (exact arithmetic otherwise), and the engine may be off from the exact logits by at most
# these factors times what that rounding alone costs (two draws of the same rounding noise
# differ by less than this; the largest of a few thousand elements varies more than the rms).
BF16_RMS_FACTOR = 2.0
BF16_MAX_FACTOR = 2.5


def assert_close(got: np.ndarray, want: np.ndarray, dtype: str, what: str = "", noise: np.ndarray = None) -> None:
    """`noise`: for bfloat16, the oracle's logits with bfloat16 storage of activations."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    assert got.shape == want.shape, f"{what}: shape {got.shape} vs {want.shape}"
    assert np.isfinite(got).all(), f"{what}: non-finite logits"
    diff = np.abs(got - want)
    if dtype == "float32":
        worst = diff.max()
        if worst > F32_ATOL:
            i = np.unravel_index(diff.argmax(), diff.shape)
            first = np.argwhere((diff > F32_ATOL).any(axis=-1)).ravel()[:5] if diff.ndim == 2 else []
            raise AssertionError(f"{what}: max |diff| {worst:.3e} > {F32_ATOL} at {i}; first bad rows {list(first)}")
    else:
        assert noise is not None, "bfloat16 comparisons need the oracle's bfloat16-storage logits"
        base = np.abs(np.asarray(noise, np.float64) - want)
        lim_max = BF16_MAX_FACTOR * base.max()
        lim_rms = BF16_RMS_FACTOR * np.sqrt((base ** 2).mean())
        rms = np.sqrt((diff ** 2).mean())
        if diff.max() > lim_max or rms > lim_rms:
            first = np.argwhere((diff > lim_max).any(axis=-1)).ravel()[:5] if diff.ndim == 2 else []
            raise AssertionError(f"{what}: max |diff| {diff.max():.3e} (limit {lim_max:.3e}), rms {rms:.3e} "
                                 f"(limit {lim_rms:.3e}); first bad rows {list(first)}")


def check_logits(got, folder: str, tokens: Sequence[int], dtype: str, what: str = "") -> None:
    noise = oracle_logits_bf16_storage(folder, tokens) if dtype == "bfloat16" else None
    assert_close(got, oracle_logits(folder, tokens), dtype, what, noise)


# ---- cutting a request into steps -----------------------------------------------
def cut_whole(n: int) -> List[int]:
    return [n]


def cut_tail_decoded(n: int, tail: int = 32) -> List[int]:
    tail = min(tail, n - 1) if n > 1 else 0
    return ([n - tail] if n - tail > 0 else []) + [1] * tail


def cut_changing(n: int, seed: int) -> List[int]:
    sizes = [7, 2, 16, 3, 2, 33, 5, 2, 64, 9, 2, 17]
    rng = np.random.default_rng(seed)
    out, left, i = [], n, int(rng.integers(0, len(sizes)))
    while left > 0:
        s = min(sizes[i % len(sizes)], left)
        if left - s == 1:   # never leave a single token: the smallest portion tested is two
            s = left if left <= 3 else s - 1
        out.append(s)
        left -= s
        i += 1
    return out
