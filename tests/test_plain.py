"""Pins for the plain implementation: vectors that the reference's own tests
hold, special cases that reduce to a library routine, and invariants.  Each is
chosen so that one plausible mistake fails it (named in the test)."""
import math

import numpy as np
import pytest

import plain_llama as P


def rnd(*shape, seed=0, scale=1.0):
    return np.random.default_rng(seed).standard_normal(shape) * scale


# ---- matrix product -------------------------------------------------------
def test_linear_is_x_times_w_transposed():
    # crates/allpaca-cpu/src/kernels.rs:2551-2560 holds matmul [[1,2],[3,4]].[[5,6],[7,8]]
    # = 19,22,43,50 for the plain product; W is stored [out,in], so the same
    # numbers come from W = B^T.  A product with W untransposed gives 17,23,39,53.
    a = np.array([[1.0, 2.0], [3.0, 4.0]])
    b = np.array([[5.0, 6.0], [7.0, 8.0]])
    assert np.allclose(P.linear(a, b.T), [[19, 22], [43, 50]])
    assert not np.allclose(P.linear(a, b), [[19, 22], [43, 50]])


# ---- rms norm -------------------------------------------------------------
def test_rmsnorm_reference_vector():
    # crates/allpaca-cpu/src/kernels.rs:2571-2578
    out = P.rms_norm(np.array([3.0, 4.0]), np.ones(2), 1e-6)
    assert abs(out[0] - 3.0 / math.sqrt(12.5 + 1e-6)) < 1e-12


def test_rmsnorm_eps_is_inside_the_root_and_added_to_the_mean():
    x = np.array([1e-3, -1e-3, 2e-3, 0.0])
    eps = 1e-2
    want = x / math.sqrt((x * x).mean() + eps)
    assert np.allclose(P.rms_norm(x, np.ones(4), eps), want, rtol=1e-12)
    # eps outside the root, or added to the sum, differ by far more than 1e-12
    assert not np.allclose(want, x / (math.sqrt((x * x).mean()) + eps), rtol=1e-3)
    assert not np.allclose(want, x / math.sqrt(((x * x).sum() + eps) / 4), rtol=1e-3)
    assert np.all(P.rms_norm(np.zeros(4), np.ones(4), 1e-5) == 0.0)  # no NaN at x = 0


def test_rmsnorm_weight_multiplies_plainly_not_one_plus_w():
    x = rnd(5, 8)
    w = rnd(8, seed=1)
    base = P.rms_norm(x, np.ones(8), 1e-5)
    assert np.allclose(P.rms_norm(x, w, 1e-5), base * w)
    assert np.allclose(P.rms_norm(x, np.zeros(8), 1e-5), 0.0)
    assert np.allclose((base * base).mean(axis=-1), 1.0, atol=1e-4)
    assert np.allclose(P.rms_norm(7.0 * x, w, 0.0), P.rms_norm(x, w, 0.0))


# ---- rope -----------------------------------------------------------------
def test_rope_identity_norm_pairing_and_sign():
    d = 8
    inv = P.rope_inv_freq(d, 10000.0)
    x = rnd(3, 2, d)
    assert np.allclose(P.rope_neox(x, [0, 0, 0], inv), x)  # pos 0 is the identity
    y = P.rope_neox(x, [3, 5, 11], inv)
    assert np.allclose((y * y).sum(-1), (x * x).sum(-1))  # kernels.rs:2581-2587
    # pairing: only (i, i + d/2) mix.  A unit vector at index 1 moves to {1, 5} only;
    # adjacent pairing would move it to {0, 1}.
    e = np.zeros((1, 1, d))
    e[0, 0, 1] = 1.0
    r = P.rope_neox(e, [2], inv)[0, 0]
    assert set(np.nonzero(np.abs(r) > 1e-12)[0]) == {1, 5}
    # sign: x_i' = a cos - b sin, x_{i+half}' = a sin + b cos
    ang = 2 * inv[1]
    assert np.isclose(r[1], math.cos(ang)) and np.isclose(r[5], math.sin(ang))
    # inverse rotation restores the input (kernels.rs:2590-2603 for the offset form)
    back = P.rope_neox(y, [3, 5, 11], -inv)
    assert np.allclose(back, x)


def test_rope_frequency_stream():
    # theta_scale = theta^(-2/d); angle_i = pos * theta_scale^i (kernels.rs:640-683)
    d, theta = 16, 500000.0
    inv = P.rope_inv_freq(d, theta)
    scale = theta ** (-2.0 / d)
    assert np.allclose(inv, [scale**i for i in range(d // 2)])
    assert inv[0] == 1.0 and np.all(np.diff(inv) < 0)


def test_rope_scores_depend_on_distance_only():
    d = 16
    inv = P.rope_inv_freq(d, 10000.0, dict(factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                           original_max_position_embeddings=64))
    q, k = rnd(1, 1, d, seed=3), rnd(1, 1, d, seed=4)
    def score(pq, pk):
        return float((P.rope_neox(q, [pq], inv) * P.rope_neox(k, [pk], inv)).sum())
    assert np.isclose(score(9, 4), score(109, 104))
    assert np.isclose(score(9, 4), score(5, 0))
    assert not np.isclose(score(9, 4), score(9, 5))


def test_llama3_scaling_regions():
    scaling = dict(factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0, original_max_position_embeddings=64)
    d, theta = 32, 500000.0
    base = P.rope_inv_freq(d, theta)
    sc = P.rope_inv_freq(d, theta, scaling)
    lam = 2 * math.pi / base
    L, lo, hi = 64.0, 1.0, 4.0
    high, low = lam < L / hi, lam > L / lo
    mid = ~high & ~low
    assert high.any() and low.any() and mid.any()  # this table has all three regions
    assert np.array_equal(sc[high], base[high])
    assert np.allclose(sc[low], base[low] / 8.0, rtol=1e-15)
    assert np.all(sc[mid] < base[mid]) and np.all(sc[mid] > base[mid] / 8.0)
    assert np.all(np.diff(sc) < 0)  # still monotone
    one = dict(scaling, factor=1.0)
    assert np.allclose(P.rope_inv_freq(d, theta, one), base, rtol=1e-15)
    # continuity at both borders: a wavelength just inside the blend is close to its neighbour rule
    def at(lam_value):
        th = 1.0  # inv_freq[0] = 1 for any theta; use head_dim 2 and scale wavelength through L
        inv = P.rope_inv_freq(2, th, dict(scaling, original_max_position_embeddings=lam_value))
        return inv[0]
    # inv_freq = 1 -> lam = 2*pi.  L/hi = lam  <=> L = 4*lam ; L/lo = lam <=> L = lam
    lam1 = 2 * math.pi
    assert np.isclose(at(4 * lam1 * (1 + 1e-9)), at(4 * lam1 * (1 - 1e-9)), rtol=1e-6)
    assert np.isclose(at(lam1 * (1 + 1e-9)), at(lam1 * (1 - 1e-9)), rtol=1e-6)


def test_llama3_scaling_inside_the_blended_band():
    """The regions, monotony and continuity above hold for a blend that is linear in the wavelength as well; the
    rule blends linearly in L / wavelength.  The band's values as numbers (factor by which a pair's frequency is
    multiplied), worked out by hand for the two tiny tables and for the table of the 8B models: with
    r = L * inv_freq / (2 pi), s = (r - low) / (high - low), the factor is (1 - s) / factor + s.  Tiny B, pair 2:
    inv_freq = 500000^(-2/16) = 0.19391, r = 64 * 0.19391 / 6.28319 = 1.97512, s = 0.32504, factor
    0.67496 / 8 + 0.32504 = 0.40941 (the full digits below).  A blend linear in the wavelength would give
    0.70 there.  The reference has no text for this rule; both the plain implementation and the engine's table are
    held to these numbers."""
    from allpaca_amd.parts.rope import inverse_frequencies
    cases = [
        (32, 500000.0, dict(factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0, original_max_position_embeddings=64),
         {2: 0.4094569168877563}, 2, 3),
        (48, 250000.0, dict(factor=4.0, low_freq_factor=1.0, high_freq_factor=2.0, original_max_position_embeddings=32),
         {2: 0.8558231322063858, 3: 0.30777214364746464}, 2, 4),
        (128, 500000.0, dict(factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0, original_max_position_embeddings=8192),
         {29: 0.8281684118371798, 30: 0.6437431331275951, 31: 0.49350712273197106, 32: 0.37112227951784466,
          33: 0.2714254770727862, 34: 0.19021074364065016}, 29, 35),
    ]
    for d, theta, scaling, band, first, end in cases:
        base = np.array([theta ** (-2.0 * i / d) for i in range(d // 2)])
        for table in (P.rope_inv_freq(d, theta, scaling), inverse_frequencies(d, theta, dict(scaling, rope_type="llama3"))):
            ratio = np.asarray(table, np.float64) / base
            for i, want in band.items():
                assert abs(ratio[i] - want) <= 1e-12 * want, (d, i, ratio[i], want)
            assert np.allclose(ratio[:first], 1.0, rtol=1e-13) and np.allclose(ratio[end:], 1.0 / scaling["factor"], rtol=1e-13)
            assert sorted(band) == list(range(first, end))     # the band is exactly these pairs


# ---- attention ------------------------------------------------------------
def test_attention_single_key_and_uniform_keys():
    d = 4
    q = rnd(1, 2, d)
    k = rnd(1, 1, d, seed=1)
    v = rnd(1, 1, d, seed=2)
    out = P.attention(q, k, v, 2, 1)
    assert np.allclose(out[0, 0], v[0, 0]) and np.allclose(out[0, 1], v[0, 0])
    k5 = np.repeat(k, 5, axis=0)
    v5 = rnd(5, 1, d, seed=5)
    q5 = np.repeat(q, 5, axis=0)
    out = P.attention(q5, k5, v5, 2, 1, causal=False)
    assert np.allclose(out[0, 0], v5[:, 0].mean(0))


def test_attention_reduces_to_softmax_qk_v():
    # no rotation, no mask, one head: softmax(Q K^T / sqrt(d)) V
    d, n = 8, 6
    q, k, v = rnd(n, 1, d, seed=1), rnd(n, 1, d, seed=2), rnd(n, 1, d, seed=3)
    s = q[:, 0] @ k[:, 0].T / math.sqrt(d)
    p = np.exp(s - s.max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)
    assert np.allclose(P.attention(q, k, v, 1, 1, causal=False)[:, 0], p @ v[:, 0])
    # scale: 1/sqrt(d), not 1/d and not missing
    assert not np.allclose(P.attention(q, k, v, 1, 1, causal=False)[:, 0],
                           (lambda z: (np.exp(z) / np.exp(z).sum(-1, keepdims=True)) @ v[:, 0])(q[:, 0] @ k[:, 0].T))


def test_attention_grouping_is_consecutive():
    # heads 0,1 read kv head 0 and heads 2,3 read kv head 1 (h // reps), not h % Hk
    d = 4
    q = np.ones((1, 4, d))
    k = np.zeros((1, 2, d))
    v = np.stack([np.full((1, d), 1.0), np.full((1, d), 2.0)], axis=1)  # [1, 2, d]
    out = P.attention(q, k, v, 4, 2)
    assert np.allclose(out[0, :, 0], [1, 1, 2, 2])


def test_attention_causal_is_bottom_right_aligned():
    d, n_kv, n_q = 4, 7, 3
    k, v = rnd(n_kv, 1, d, seed=1), rnd(n_kv, 1, d, seed=2)
    qfull = rnd(n_kv, 1, d, seed=3)
    full = P.attention(qfull, k, v, 1, 1)
    part = P.attention(qfull[-n_q:], k, v, 1, 1)  # the last rows over the whole history
    assert np.allclose(part, full[-n_q:])
    # row 0 of the full pass sees key 0 only
    assert np.allclose(full[0, 0], v[0, 0])


def test_attention_finds_a_far_key():
    # one key among hundreds matches the query with a large score: the output is its value
    d, n = 16, 300
    k = rnd(n, 1, d, seed=1, scale=0.1)
    v = rnd(n, 1, d, seed=2)
    q = rnd(n, 1, d, seed=3, scale=0.1)
    k[17, 0] = 0.0
    k[17, 0, 3] = 40.0
    q[-1, 0] = 0.0
    q[-1, 0, 3] = 40.0
    out = P.attention(q, k, v, 1, 1)
    assert np.allclose(out[-1, 0], v[17, 0], atol=1e-6)


def test_attention_window():
    d, n = 4, 9
    q, k, v = rnd(n, 1, d, seed=1), rnd(n, 1, d, seed=2), rnd(n, 1, d, seed=3)
    w = 3
    out = P.attention(q, k, v, 1, 1, window=w)
    for i in range(n):
        lo = max(0, i - w + 1)
        want = P.attention(q[i : i + 1], k[lo : i + 1], v[lo : i + 1], 1, 1)
        assert np.allclose(out[i], want[0])
    assert np.allclose(P.attention(q, k, v, 1, 1, window=n), P.attention(q, k, v, 1, 1))


def test_softmax_rows_sum_to_one():
    # kernels.rs:2563-2568
    p = P.softmax_rows(np.array([[1.0, 2.0, 3.0]]))
    assert abs(p.sum() - 1.0) < 1e-12
    assert np.allclose(P.softmax_rows(np.full((1, 4), -np.inf)), 0.25)


# ---- feed-forward ---------------------------------------------------------
def test_silu():
    assert P.silu(0.0) == 0.0
    assert np.isclose(P.silu(30.0), 30.0)
    z = np.linspace(-6, 6, 25)
    assert np.allclose(P.silu(z) - P.silu(-z), z)
    assert np.allclose(P.silu(z), z * (1 / (1 + np.exp(-z))))


def test_swiglu_gate_is_the_activated_branch():
    h = rnd(3, 5)
    wg, wu, wd = rnd(7, 5, seed=1), rnd(7, 5, seed=2), rnd(5, 7, seed=3)
    want = (P.silu(h @ wg.T) * (h @ wu.T)) @ wd.T
    assert np.allclose(P.swiglu(h, wg, wu, wd), want)
    assert not np.allclose(P.swiglu(h, wu, wg, wd), want)  # swapped branches differ


# ---- stack ----------------------------------------------------------------
def tiny_cfg(**over):
    cfg = dict(architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=50, hidden_size=24,
               num_hidden_layers=2, num_attention_heads=3, num_key_value_heads=1, head_dim=8,
               intermediate_size=40, rms_norm_eps=1e-5, rope_theta=10000.0, tie_word_embeddings=False,
               max_position_embeddings=64)
    cfg.update(over)
    return cfg


def tiny_weights(cfg, seed=0, std=0.3):
    rng = np.random.default_rng(seed)
    H, Hk, d = P.llama_dims(cfg)
    D, F, V = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    w = {"model.embed_tokens.weight": rng.standard_normal((V, D)) * std,
         "model.norm.weight": 1 + 0.1 * rng.standard_normal(D)}
    for l in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{l}."
        w[p + "input_layernorm.weight"] = 1 + 0.1 * rng.standard_normal(D)
        w[p + "post_attention_layernorm.weight"] = 1 + 0.1 * rng.standard_normal(D)
        w[p + "self_attn.q_proj.weight"] = rng.standard_normal((H * d, D)) * std
        w[p + "self_attn.k_proj.weight"] = rng.standard_normal((Hk * d, D)) * std
        w[p + "self_attn.v_proj.weight"] = rng.standard_normal((Hk * d, D)) * std
        w[p + "self_attn.o_proj.weight"] = rng.standard_normal((D, H * d)) * std
        w[p + "mlp.gate_proj.weight"] = rng.standard_normal((F, D)) * std
        w[p + "mlp.up_proj.weight"] = rng.standard_normal((F, D)) * std
        w[p + "mlp.down_proj.weight"] = rng.standard_normal((D, F)) * std
    if not cfg.get("tie_word_embeddings"):
        w["lm_head.weight"] = rng.standard_normal((V, D)) * std
    return w


def test_zero_output_projections_make_layers_the_identity():
    cfg = tiny_cfg()
    w = tiny_weights(cfg)
    for l in range(2):
        w[f"model.layers.{l}.self_attn.o_proj.weight"][:] = 0
        w[f"model.layers.{l}.mlp.down_proj.weight"][:] = 0
    toks = [3, 9, 3, 11]
    want = P.rms_norm(w["model.embed_tokens.weight"][toks], w["model.norm.weight"], 1e-5) @ w["lm_head.weight"].T
    assert np.allclose(P.llama_forward(cfg, w, toks), want)


def test_causality_and_prefix_property():
    cfg = tiny_cfg()
    w = tiny_weights(cfg)
    toks = [1, 2, 3, 4, 5, 6, 7]
    full = P.llama_forward(cfg, w, toks)
    assert np.allclose(P.llama_forward(cfg, w, toks[:4]), full[:4])
    other = P.llama_forward(cfg, w, toks[:4] + [9, 9, 9])
    assert np.allclose(other[:4], full[:4]) and not np.allclose(other[4:], full[4:])


def test_shift_of_all_positions_changes_nothing():
    cfg = tiny_cfg(rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0,
                                     high_freq_factor=4.0, original_max_position_embeddings=16))
    w = tiny_weights(cfg, seed=2)
    toks = [4, 8, 15, 16, 23, 42]
    a = P.llama_forward(cfg, w, toks)
    b = P.llama_forward(cfg, w, toks, positions=np.arange(6) + 37)
    assert np.allclose(a, b, atol=1e-9)
    c = P.llama_forward(cfg, w, toks, positions=np.arange(6) * 2)  # distances change -> logits change
    assert not np.allclose(a, c, atol=1e-6)


def test_norm_sits_before_the_mixer_and_residual_skips_it():
    # one layer, by hand
    cfg = tiny_cfg(num_hidden_layers=1, num_attention_heads=1, num_key_value_heads=1, head_dim=24)
    w = tiny_weights(cfg, seed=5)
    toks = [7]
    x = w["model.embed_tokens.weight"][toks]
    p = "model.layers.0."
    h = P.rms_norm(x, w[p + "input_layernorm.weight"], 1e-5)
    v = h @ w[p + "self_attn.v_proj.weight"].T  # one token: attention output is its own value
    x1 = x + v @ w[p + "self_attn.o_proj.weight"].T
    h2 = P.rms_norm(x1, w[p + "post_attention_layernorm.weight"], 1e-5)
    x2 = x1 + P.swiglu(h2, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    want = P.rms_norm(x2, w["model.norm.weight"], 1e-5) @ w["lm_head.weight"].T
    assert np.allclose(P.llama_forward(cfg, w, toks), want)


def test_tied_head_uses_the_embedding_matrix():
    cfg = tiny_cfg(tie_word_embeddings=True)
    w = tiny_weights(cfg)
    assert "lm_head.weight" not in w
    logits, hN = P.llama_forward(cfg, w, [5, 6], return_hidden=True)
    assert np.allclose(logits, hN @ w["model.embed_tokens.weight"].T)


# ---- sampler --------------------------------------------------------------
def test_argmax_first_maximum_wins():
    assert P.argmax([1.0, 5.0, 5.0, 2.0]) == 1
    assert P.argmax([-np.inf, -np.inf]) == 0


def test_sampler_cases():
    lg = np.array([0.1, 2.0, -1.0, 2.0, 0.5], np.float32)
    assert P.sample(lg, 0.0, 40, 0.95, 0.7) == 1  # greedy
    assert P.sample(np.full(5, np.nan, np.float32), 0.8, 40, 0.95, 0.3) == 0  # degenerate
    cand, _ = P.sample_candidates(lg, 1.0, 2, 1.0)
    assert [c[0] for c in cand] == [1, 3]  # top-k, ties by lower id
    assert np.isclose(sum(p for _, p in cand), 1.0)
    cand, _ = P.sample_candidates(lg, 1.0, 0, 1.0)
    assert [c[0] for c in cand] == [0, 1, 2, 3, 4]  # no filter: id order
    pr = np.exp(lg.astype(np.float64))
    pr /= pr.sum()
    assert np.allclose([p for _, p in cand], pr)
    cand, _ = P.sample_candidates(lg, 1.0, 0, 0.5)
    assert [c[0] for c in cand] == [1, 3]  # 0.37 + 0.37 >= 0.5
    cand, _ = P.sample_candidates(lg, 1.0, 0, 0.3)
    assert [c[0] for c in cand] == [1]
    # the walk: r just under the first probability picks the first, just over the second
    cand, _ = P.sample_candidates(lg, 0.7, 0, 1.0)
    p0 = cand[0][1]
    assert P.sample(lg, 0.7, 0, 1.0, p0 * 0.999) == 0
    assert P.sample(lg, 0.7, 0, 1.0, p0 * 1.001) == 1
    assert P.sample(lg, 0.7, 0, 1.0, 0.9999999) == 4


def test_sampler_frequencies_match_softmax():
    lg = np.array([0.0, 1.0, 2.0, -1.0], np.float32)
    T = 0.8
    rng = np.random.default_rng(0)
    n = 20000
    counts = np.zeros(4)
    for r in rng.random(n):
        counts[P.sample(lg, T, 0, 1.0, r)] += 1
    p = np.exp(lg / T)
    p /= p.sum()
    chi2 = ((counts - n * p) ** 2 / (n * p)).sum()
    assert chi2 < 16.27  # 3 degrees of freedom, p = 0.001


def test_uniform_numbers_of_many_rows_equal_the_ones_of_each_row():
    """The sampler draws a step's uniform numbers for all rows at once (64-bit arithmetic that wraps in numpy); they
    are the numbers `uniform_for` gives row by row with Python integers."""
    from allpaca_amd.sampling.sampler import uniform_for, uniforms_for
    rng = np.random.default_rng(0)
    seeds = [int(x) for x in rng.integers(0, 2 ** 63, size=500)] + [0, 1, 2 ** 64 - 1, 2 ** 63, 12345]
    idx = [int(x) for x in rng.integers(0, 1 << 20, size=len(seeds))]
    one = np.asarray([uniform_for(s, i) for s, i in zip(seeds, idx)], dtype=np.float32)
    many = uniforms_for(seeds, idx)
    assert many.dtype == np.float32 and np.array_equal(one, many) and (many >= 0).all() and (many < 1).all()
