"""A plain, slow implementation of the dense llama decoder and of the sampler.

Whole sequences, no cache, no batching, one function for each part, NumPy in
float64 (inputs are widened exactly).  It shares no code with `allpaca_amd`:
it has its own safetensors reader and its own config reading.  Every function
cites the reference text (paths relative to the reference checkout) that fixes
its formula.  The reference is read, not run.
"""
from __future__ import annotations

import json
import math
import os
import struct

import numpy as np

F64 = np.float64


# ---------------------------------------------------------------------------
# file reading (own code: header JSON + raw little-endian payload)
# ---------------------------------------------------------------------------
def _bf16_to_f32(raw: np.ndarray) -> np.ndarray:
    # bf16 is the upper half of an IEEE float32
    # (crates/allpaca-safetensors/src/parser.rs:16-46: BF16 widened to f32).
    return (raw.astype(np.uint32) << 16).view(np.float32)


def read_safetensors(path: str) -> dict:
    """name -> float64/int64 ndarray.  Layout: 8-byte LE header length, JSON
    header {name: {dtype, shape, data_offsets}}, payload
    (crates/allpaca-safetensors/src/parser.rs:93-160)."""
    with open(path, "rb") as f:
        blob = f.read()
    (hlen,) = struct.unpack("<Q", blob[:8])
    header = json.loads(blob[8 : 8 + hlen].decode("utf-8"))
    base = 8 + hlen
    out = {}
    for name, info in header.items():
        if name == "__metadata__":
            continue
        lo, hi = info["data_offsets"]
        raw = blob[base + lo : base + hi]
        dt = info["dtype"]
        if dt == "F32":
            arr = np.frombuffer(raw, dtype="<f4").astype(F64)
        elif dt == "BF16":
            arr = _bf16_to_f32(np.frombuffer(raw, dtype="<u2")).astype(F64)
        elif dt == "F16":
            arr = np.frombuffer(raw, dtype="<f2").astype(F64)
        elif dt == "I32":
            arr = np.frombuffer(raw, dtype="<i4").astype(np.int64)
        else:
            raise ValueError(f"plain reader: dtype {dt} of {name}")
        out[name] = arr.reshape(info["shape"])
    return out


def read_model_folder(folder: str):
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    return cfg, read_safetensors(os.path.join(folder, "model.safetensors"))


# ---------------------------------------------------------------------------
# parts
# ---------------------------------------------------------------------------
def embedding(table: np.ndarray, tokens) -> np.ndarray:
    """x0 = E[token], a row copy, no scale for llama
    (crates/allpaca-core/src/model.rs:8301-8311)."""
    return np.asarray(table, F64)[np.asarray(tokens, np.int64)]


def linear(x: np.ndarray, w: np.ndarray) -> np.ndarray:
    """y = x . W^T with W stored [out, in]
    (crates/allpaca-cpu/src/kernels.rs:97-128)."""
    return np.asarray(x, F64) @ np.asarray(w, F64).T


def rms_norm(x: np.ndarray, weight: np.ndarray, eps: float) -> np.ndarray:
    """ss = sum x^2; inv = 1/sqrt(ss/D + eps); out = x*inv*w.  eps is added to
    the mean inside the root; the weight multiplies after normalisation
    (crates/allpaca-cpu/src/kernels.rs:492-507)."""
    x = np.asarray(x, F64)
    ss = (x * x).sum(axis=-1, keepdims=True)
    inv = 1.0 / np.sqrt(ss / x.shape[-1] + eps)
    return x * inv * np.asarray(weight, F64)


def rope_inv_freq(head_dim: int, theta: float, scaling: dict | None = None) -> np.ndarray:
    """inv_freq[i] = theta^(-2i/d), i < d/2: the reference's NeoX stream
    `theta_scale = theta^(-2/n_rot)`, angle_i = pos * theta_scale^i
    (crates/allpaca-cpu/src/kernels.rs:640-683).

    Llama-3 frequency scaling has no text in the reference (its llama path
    reads rope_theta only, crates/allpaca-core/src/model.rs:181-274); the rule
    is the published one: wavelength lam = 2*pi/inv_freq; lam < L/hi keeps the
    frequency, lam > L/lo divides it by `factor`, between them a linear blend
    in s = (L/lam - lo)/(hi - lo)."""
    half = head_dim // 2
    inv = np.array([theta ** (-2.0 * i / head_dim) for i in range(half)], F64)
    if not scaling:
        return inv
    f = float(scaling["factor"])
    lo = float(scaling["low_freq_factor"])
    hi = float(scaling["high_freq_factor"])
    L = float(scaling["original_max_position_embeddings"])
    out = inv.copy()
    for i in range(half):
        lam = 2.0 * math.pi / inv[i]
        if lam < L / hi:
            out[i] = inv[i]
        elif lam > L / lo:
            out[i] = inv[i] / f
        else:
            s = (L / lam - lo) / (hi - lo)
            out[i] = (1.0 - s) * inv[i] / f + s * inv[i]
    return out


def rope_neox(x: np.ndarray, positions, inv_freq: np.ndarray) -> np.ndarray:
    """x: [T, n_heads, d].  Pairs (i, i + d/2) of every head turn by
    pos*inv_freq[i]:  x_i' = a cos - b sin,  x_{i+d/2}' = a sin + b cos
    (crates/allpaca-cpu/src/kernels.rs:676-682; the HF safetensors path sets
    rope_neox, crates/allpaca-core/src/model.rs:7937)."""
    x = np.asarray(x, F64)
    half = x.shape[-1] // 2
    ang = np.asarray(positions, F64)[:, None] * np.asarray(inv_freq, F64)[None, :]  # [T, half]
    cos, sin = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
    a, b = x[..., :half], x[..., half:]
    return np.concatenate([a * cos - b * sin, a * sin + b * cos], axis=-1)


def softmax_rows(s: np.ndarray) -> np.ndarray:
    """m = max; e = exp(s - m); p = e/sum e; a row with no finite score is
    uniform, a guard only (crates/allpaca-cpu/src/kernels.rs:746-778)."""
    s = np.asarray(s, F64)
    m = s.max(axis=-1, keepdims=True)
    safe = np.where(np.isfinite(m), m, 0.0)
    e = np.exp(s - safe)
    e = np.where(np.isfinite(m), e, 1.0)
    return e / e.sum(axis=-1, keepdims=True)


def attention(q, k, v, n_heads: int, n_kv_heads: int, causal: bool = True, window: int | None = None):
    """q: [n_q, H, d]; k, v: [n_kv, Hk, d] -> [n_q, H, d].
    Query head h reads kv head h // (H/Hk) (consecutive heads share);
    score = (q.k) * (1/sqrt(d)), the scale on the finished dot product;
    causal mask bottom-right aligned: key t is hidden when t > qi + (n_kv - n_q)
    (crates/allpaca-cpu/src/kernels.rs:293-356).  `window` (not used by llama)
    hides keys with t <= qpos - window."""
    q, k, v = np.asarray(q, F64), np.asarray(k, F64), np.asarray(v, F64)
    n_q, n_kv, d = q.shape[0], k.shape[0], q.shape[-1]
    assert n_heads % n_kv_heads == 0
    reps = n_heads // n_kv_heads
    scale = 1.0 / math.sqrt(d)
    out = np.zeros_like(q)
    for h in range(n_heads):
        kh = h // reps
        s = (q[:, h, :] @ k[:, kh, :].T) * scale  # [n_q, n_kv]
        qpos = np.arange(n_q)[:, None] + (n_kv - n_q)
        t = np.arange(n_kv)[None, :]
        if causal:
            s = np.where(t > qpos, -np.inf, s)
        if window is not None:
            s = np.where(t <= qpos - window, -np.inf, s)
        out[:, h, :] = softmax_rows(s) @ v[:, kh, :]
    return out


def silu(z):
    """silu(z) = z / (1 + exp(-z)) (crates/allpaca-cpu/src/kernels.rs:869-871)."""
    z = np.asarray(z, F64)
    return z / (1.0 + np.exp(-z))


def swiglu(h, w_gate, w_up, w_down):
    """g = h Wg^T, u = h Wu^T, a = silu(g)*u, y = a Wd^T
    (crates/allpaca-core/src/model.rs:5664-5705)."""
    return linear(silu(linear(h, w_gate)) * linear(h, w_up), w_down)


# ---------------------------------------------------------------------------
# whole model
# ---------------------------------------------------------------------------
def llama_dims(cfg: dict):
    H = cfg["num_attention_heads"]
    Hk = cfg.get("num_key_value_heads") or H
    d = cfg.get("head_dim") or cfg["hidden_size"] // H  # model.rs:366-372
    return H, Hk, d


def round_bf16(x):
    """Round to the nearest bfloat16 (ties to even), returned as float64: what storing an
    activation in bfloat16 does to it."""
    f = np.asarray(x, np.float32)
    u = f.view(np.uint32)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & np.uint32(0xFFFF0000)
    return u.view(np.float32).astype(F64)


def llama_forward(cfg: dict, w: dict, tokens, positions=None, return_hidden: bool = False, store=None):
    """Logits [T, V] of one whole sequence (crates/allpaca-core/src/model.rs:8301-8792
    in the order of the host forward): embed; per layer  h = norm(x); q,k,v;
    rope(q,k); causal attention; x += o Wo^T; h = norm(x); x += swiglu(h);
    final norm; head (tied: the embedding matrix, model.rs:8005-8009).

    `store` (e.g. `round_bf16`) is applied to every activation that a reduced-precision
    run keeps between two matrix products (normed input, q/k/v before and after
    rotation, attention output, SwiGLU output), never to the residual stream or the
    logits: it shows what such storage alone costs, with exact arithmetic otherwise."""
    st = store if store is not None else (lambda z: z)
    H, Hk, d = llama_dims(cfg)
    eps = cfg.get("rms_norm_eps", 1e-5)
    theta = cfg.get("rope_theta", 10000.0)
    inv_freq = rope_inv_freq(d, theta, cfg.get("rope_scaling"))
    T = len(tokens)
    pos = np.arange(T) if positions is None else np.asarray(positions)
    x = embedding(w["model.embed_tokens.weight"], tokens)
    for l in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{l}."
        h = st(rms_norm(x, w[p + "input_layernorm.weight"], eps))
        q = st(linear(h, w[p + "self_attn.q_proj.weight"])).reshape(T, H, d)
        k = st(linear(h, w[p + "self_attn.k_proj.weight"])).reshape(T, Hk, d)
        v = st(linear(h, w[p + "self_attn.v_proj.weight"])).reshape(T, Hk, d)
        q, k = st(rope_neox(q, pos, inv_freq)), st(rope_neox(k, pos, inv_freq))
        o = st(attention(q, k, v, H, Hk, causal=True).reshape(T, H * d))
        x = x + linear(o, w[p + "self_attn.o_proj.weight"])
        h = st(rms_norm(x, w[p + "post_attention_layernorm.weight"], eps))
        if store is None:
            x = x + swiglu(h, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
        else:
            a = st(silu(linear(h, w[p + "mlp.gate_proj.weight"])) * linear(h, w[p + "mlp.up_proj.weight"]))
            x = x + linear(a, w[p + "mlp.down_proj.weight"])
    hN = st(rms_norm(x, w["model.norm.weight"], eps))
    head = w["lm_head.weight"] if "lm_head.weight" in w else w["model.embed_tokens.weight"]
    logits = linear(hN, head)
    return (logits, hN) if return_hidden else logits


def greedy_generate(cfg: dict, w: dict, prompt, n_new: int):
    """Greedy continuation by recomputing the whole sequence each token."""
    toks = list(prompt)
    out = []
    for _ in range(n_new):
        logits = llama_forward(cfg, w, toks)
        t = argmax(logits[-1])
        out.append(t)
        toks.append(t)
    return out


# ---------------------------------------------------------------------------
# sampler
# ---------------------------------------------------------------------------
def argmax(logits) -> int:
    """First maximum wins (strict >), crates/allpaca-core/src/sampling.rs:215-225."""
    best_i, best = 0, -math.inf
    for i, v in enumerate(np.asarray(logits).tolist()):
        if v > best:
            best, best_i = v, i
    return best_i


def sample_candidates(logits, temperature: float, top_k: int, top_p: float):
    """Ordered list [(id, prob)] that the draw walks
    (crates/allpaca-core/src/sampling.rs:24-52, 227-331): all non-finite ->
    [(0,1)]; temperature <= 1e-5 -> one-hot argmax; else logits / max(T,1e-5);
    finite candidates in id order; top-k keeps the k largest sorted by logit
    descending, ties by lower id; top-p (0 <= p < 1) keeps the shortest sorted
    prefix whose probability (over the candidates left) reaches p; softmax."""
    lg = np.asarray(logits, np.float32).astype(F64)
    if not np.isfinite(lg).any():
        return [(0, 1.0)], False
    if temperature <= 1e-5:
        return [(argmax(lg), 1.0)], False
    lg = np.where(np.isfinite(lg), lg / max(temperature, 1e-5), lg)
    cand = [(i, float(v)) for i, v in enumerate(lg) if np.isfinite(v)]
    by_desc = lambda c: (-c[1], c[0])
    if top_k and len(cand) > top_k:
        cand = sorted(cand, key=by_desc)[:top_k]
    if 0.0 <= top_p < 1.0 and len(cand) > 1:
        mx = max(v for _, v in cand)
        total = sum(math.exp(v - mx) for _, v in cand)
        cand = sorted(cand, key=by_desc)
        acc = 0.0
        for i, (_, v) in enumerate(cand):
            acc += math.exp(v - mx) / total
            if acc >= top_p:
                cand = cand[: i + 1]
                break
    mx = max(v for _, v in cand)
    e = [math.exp(v - mx) for _, v in cand]
    s = sum(e)
    return [(i, x / s) for (i, _), x in zip(cand, e)], True


def sample(logits, temperature: float, top_k: int, top_p: float, r: float) -> int:
    """Draw with a given uniform r in [0,1): walk r -= p until r <= 0, else the
    last candidate (crates/allpaca-core/src/sampling.rs:55-67)."""
    cand, draws = sample_candidates(logits, temperature, top_k, top_p)
    if not draws:
        return cand[0][0]
    for i, p in cand:
        r -= p
        if r <= 0.0:
            return i
    return cand[-1][0]
