"""Each plain kernel alone against a float64 reference of the same operation,
at sizes other than the engine's (odd widths, strides, both element types)."""
import math

import numpy as np
import pytest
import torch

import plain_llama as P

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def ops():
    from allpaca_amd.kernels import ops as o
    return o


def gen(*shape, seed=0, scale=1.0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g, dtype=torch.float32) * scale).to(dtype)


def f64(t):
    return t.detach().float().cpu().numpy().astype(np.float64)


def close(got, want, atol=1e-4, rtol=1e-3):
    # the reference's own bound for a kernel against its CPU counterpart
    # (crates/allpaca-hip/src/lib.rs:17060-17063): |d| <= 1e-4 or <= 1e-3 * max(|a|, |b|)
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    d = np.abs(got - want)
    ok = (d <= atol) | (d <= rtol * np.maximum(np.abs(got), np.abs(want)))
    assert ok.all(), f"max diff {d.max():.3e} at {np.unravel_index(d.argmax(), d.shape)}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embed_and_gather(dtype):
    o = ops()
    table = gen(37, 50, seed=1, dtype=dtype).to(DEV)
    toks = torch.tensor([5, 0, 36, 5, 17], dtype=torch.int32, device=DEV)
    out = torch.empty(5, 50, dtype=torch.float32, device=DEV)
    o.embed_rows(table, toks, out)
    assert torch.equal(out.cpu(), table.float().cpu()[toks.cpu().long()])
    rows = torch.tensor([4, 1, 1], dtype=torch.int32, device=DEV)
    g = torch.empty(3, 50, dtype=torch.float32, device=DEV)
    o.gather_rows(out, rows, g)
    assert torch.equal(g.cpu(), out.cpu()[[4, 1, 1]])


@pytest.mark.parametrize("D", [2, 50, 256, 1300, 4099])
def test_rmsnorm(D):
    o = ops()
    x = gen(7, D, seed=D, scale=3.0).to(DEV)
    w = (1 + 0.1 * gen(D, seed=1)).to(DEV)
    for eps in (1e-5, 1e-2):
        out = torch.empty(7, D, dtype=torch.float32, device=DEV)
        o.rmsnorm_rows(x, w, eps, out)
        close(f64(out), P.rms_norm(f64(x), f64(w), eps), atol=1e-5, rtol=1e-5)
    outb = torch.empty(7, D, dtype=torch.bfloat16, device=DEV)
    o.rmsnorm_rows(x, w, 1e-5, outb)
    close(f64(outb), P.rms_norm(f64(x), f64(w), 1e-5), atol=1e-5, rtol=2.0 ** -8)
    rows = torch.tensor([6, 0], dtype=torch.int32, device=DEV)
    sel = torch.empty(2, D, dtype=torch.float32, device=DEV)
    o.rmsnorm_rows(x, w, 1e-5, sel, rows)
    close(f64(sel), P.rms_norm(f64(x)[[6, 0]], f64(w), 1e-5), atol=1e-5, rtol=1e-5)


def test_rmsnorm_reference_vector_and_zero():
    o = ops()
    x = torch.tensor([[3.0, 4.0], [0.0, 0.0]], device=DEV)
    out = torch.empty_like(x)
    o.rmsnorm_rows(x, torch.ones(2, device=DEV), 1e-6, out)  # crates/allpaca-cpu/src/kernels.rs:2571-2578
    assert abs(out[0, 0].item() - 3.0 / math.sqrt(12.5 + 1e-6)) < 1e-6
    assert out[1].abs().max().item() == 0.0


@pytest.mark.parametrize("M,N,K", [(3, 5, 13), (2, 2100, 2003), (1, 1, 1), (70, 129, 65), (64, 64, 16)])
def test_gemm_plain(M, N, K):
    # shapes of crates/allpaca-cpu/src/kernels.rs:2486-2504 and tile-edge cases
    o = ops()
    a, w = gen(M, K, seed=1).to(DEV), gen(N, K, seed=2).to(DEV)
    out = torch.empty(M, N, device=DEV)
    o.gemm_plain(a, w, out)
    want = f64(a) @ f64(w).T
    d = np.abs(f64(out) - want)
    assert (d <= 1e-4 * (1 + np.abs(want))).all()
    acc = gen(M, N, seed=3).to(DEV)
    before = f64(acc)
    o.gemm_plain(a, w, acc, accumulate=True)
    assert (np.abs(f64(acc) - (before + want)) <= 1e-4 * (1 + np.abs(want))).all()


def test_gemm_plain_2x2_vector():
    o = ops()
    a = torch.tensor([[1.0, 2.0], [3.0, 4.0]], device=DEV)
    bT = torch.tensor([[5.0, 7.0], [6.0, 8.0]], device=DEV)  # W = B^T
    out = torch.empty(2, 2, device=DEV)
    o.gemm_plain(a, bT, out)
    assert out.cpu().tolist() == [[19.0, 22.0], [43.0, 50.0]]  # crates/allpaca-cpu/src/kernels.rs:2551-2560


def test_gemm_plain_rows_together_equal_each_row_alone():
    # crates/allpaca-cpu/src/kernels.rs:2506-2525, bit for bit
    o = ops()
    for M, N, K in [(7, 2100, 1203), (5, 37, 64), (130, 70, 33)]:
        a, w = gen(M, K, seed=3).to(DEV), gen(N, K, seed=4).to(DEV)
        tog = torch.empty(M, N, device=DEV)
        o.gemm_plain(a, w, tog)
        for r in (0, M // 2, M - 1):
            alone = torch.empty(1, N, device=DEV)
            o.gemm_plain(a[r:r + 1], w, alone)
            assert torch.equal(alone[0], tog[r])


def test_gemm_plain_mixed_types_and_strides():
    o = ops()
    big = gen(9, 100, seed=5).to(DEV)
    a = big[:, 10:43]                       # a strided view
    w = gen(21, 33, seed=6, dtype=torch.bfloat16).to(DEV)
    out = torch.empty(9, 21, dtype=torch.bfloat16, device=DEV)
    o.gemm_plain(a, w, out)
    close(f64(out), f64(a) @ f64(w).T, atol=1e-4, rtol=2.0 ** -8)


def test_silu_mul_and_add():
    o = ops()
    F = 77
    gu = gen(5, 2 * F, seed=7, scale=3.0).to(DEV)
    out = torch.empty(5, F, device=DEV)
    o.silu_mul(gu, out)
    g = f64(gu)
    close(f64(out), P.silu(g[:, :F]) * g[:, F:], atol=1e-6, rtol=1e-5)
    z = torch.tensor([[0.0, 30.0, 1.0, 1.0]], device=DEV)  # silu(0) = 0, silu(30) ~ 30
    o2 = torch.empty(1, 2, device=DEV)
    o.silu_mul(z, o2)
    assert o2[0, 0].item() == 0.0 and abs(o2[0, 1].item() - 30.0) < 1e-4
    acc = gen(5, F, seed=8).to(DEV)
    y = gen(5, F, seed=9, dtype=torch.bfloat16).to(DEV)
    want = f64(acc) + f64(y)
    o.add_into(acc, y)
    close(f64(acc), want, atol=1e-6, rtol=1e-6)


def make_cache(n_seq_tokens, Hk, d, P_, dtype, seed=0, shuffle=True, stale=0.0, loud=None):
    """Random keys/values for sequences of the given lengths laid into pages in a shuffled order.  `stale`: what
    the slots beyond a sequence's last position and the three pages that belong to no sequence hold.  `loud`:
    (sequence, position, factor): that key is multiplied by the factor, so that its scores dwarf all others."""
    rng = np.random.default_rng(seed)
    n_blocks = [-(-n // P_) for n in n_seq_tokens]
    total = sum(n_blocks)
    ids = rng.permutation(total + 3) if shuffle else np.arange(total + 3)
    cache = torch.full((total + 3, 2, Hk, P_, d), stale, dtype=dtype)
    bt = np.zeros((len(n_seq_tokens), max(n_blocks)), np.int32)
    ks, vs = [], []
    at = 0
    for s, n in enumerate(n_seq_tokens):
        k = gen(n, Hk, d, seed=seed * 100 + 2 * s, dtype=dtype)
        v = gen(n, Hk, d, seed=seed * 100 + 2 * s + 1, dtype=dtype)
        if loud is not None and loud[0] == s:
            k[loud[1]] = (k[loud[1]].float() * loud[2]).to(dtype)
        ks.append(k)
        vs.append(v)
        for b in range(n_blocks[s]):
            page = int(ids[at])
            at += 1
            bt[s, b] = page
            lo, hi = b * P_, min(n, (b + 1) * P_)
            cache[page, 0, :, : hi - lo] = k[lo:hi].permute(1, 0, 2)
            vt = torch.full((Hk, d, P_), stale, dtype=dtype)   # values lie [element][slot] inside a page
            vt[:, :, : hi - lo] = v[lo:hi].permute(1, 2, 0)
            cache[page, 1] = vt.reshape(Hk, P_, d)
    return cache.to(DEV), torch.from_numpy(bt).to(DEV), ks, vs


# shapes from the reference's attention test list (n_q, n_kv, H, Hk, d), crates/allpaca-hip/src/lib.rs:23162-23175,
# plus sizes of our own
ATTN_SHAPES = [(1, 3000, 4, 2, 128), (2, 1300, 2, 1, 64), (3, 8, 4, 1, 8), (5, 70, 6, 3, 48), (64, 64, 3, 3, 16),
               (9, 200, 5, 1, 256)]


@pytest.mark.parametrize("n_q,n_kv,H,Hk,d", ATTN_SHAPES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_paged_attention_plain(n_q, n_kv, H, Hk, d, dtype):
    o = ops()
    for P_ in (16, 7):
        cache, bt, ks, vs = make_cache([n_kv], Hk, d, P_, dtype, seed=n_kv)
        q = gen(n_q, H * d + 8, seed=11, dtype=dtype).to(DEV)  # q lives at a column offset inside wider rows
        pos = torch.arange(n_kv - n_q, n_kv, dtype=torch.int32, device=DEV)
        seg = torch.zeros(n_q, dtype=torch.int32, device=DEV)
        out = torch.empty(n_q, H * d, dtype=dtype, device=DEV)
        o.paged_attention_plain(q, 8, out, H, Hk, d, cache, P_, bt, pos, seg)
        want = P.attention(f64(q)[:, 8:].reshape(n_q, H, d), f64(ks[0]), f64(vs[0]), H, Hk)
        if dtype == torch.float32:
            close(f64(out).reshape(n_q, H, d), want)
        else:
            close(f64(out).reshape(n_q, H, d), want, atol=2e-3, rtol=2.0 ** -7)


def test_paged_attention_plain_window_and_two_sequences():
    o = ops()
    H, Hk, d, P_ = 4, 2, 32, 4
    lens = [37, 90]
    cache, bt, ks, vs = make_cache(lens, Hk, d, P_, torch.float32, seed=5)
    # rows: 3 rows of sequence 1 at positions 87..89 and one row of sequence 0 at position 36
    pos = torch.tensor([87, 88, 89, 36], dtype=torch.int32, device=DEV)
    seg = torch.tensor([1, 1, 1, 0], dtype=torch.int32, device=DEV)
    q = gen(4, H * d, seed=3).to(DEV)
    for window in (0, 10, 1, 64):
        out = torch.empty(4, H * d, device=DEV)
        o.paged_attention_plain(q, 0, out, H, Hk, d, cache, P_, bt, pos, seg, window=window)
        w = window or None
        q64 = f64(q).reshape(4, H, d)
        want1 = P.attention(q64[:3], f64(ks[1]), f64(vs[1]), H, Hk, window=w)
        want0 = P.attention(q64[3:], f64(ks[0]), f64(vs[0]), H, Hk, window=w)
        close(f64(out).reshape(4, H, d), np.concatenate([want1, want0]))


def test_paged_attention_plain_finds_a_far_key():
    o = ops()
    H, Hk, d, P_, n = 2, 1, 64, 16, 700
    cache, bt, ks, vs = make_cache([n], Hk, d, P_, torch.float32, seed=9)
    page, slot = int(bt[0, 17 // P_]), 17 % P_
    cache[page, 0, 0, slot] = 0.0
    cache[page, 0, 0, slot, 5] = 30.0
    q = torch.zeros(1, H * d, device=DEV)
    q[0, 5] = 30.0
    q[0, d + 5] = 30.0
    out = torch.empty(1, H * d, device=DEV)
    o.paged_attention_plain(q, 0, out, H, Hk, d, cache, P_, bt, torch.tensor([n - 1], dtype=torch.int32, device=DEV),
                            torch.zeros(1, dtype=torch.int32, device=DEV))
    for h in range(H):
        assert torch.allclose(out[0, h * d:(h + 1) * d].cpu(), vs[0][17, 0], atol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rope_kv_write(dtype):
    o = ops()
    H, Hk, d, P_ = 5, 2, 48, 8
    T = 6
    scaling = dict(factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0, original_max_position_embeddings=32)
    for rot in (d, 16):
        inv = P.rope_inv_freq(rot, 10000.0, scaling)
        maxpos = 64
        ang = np.arange(maxpos)[:, None] * inv[None, :]
        table = torch.from_numpy(np.stack([np.cos(ang), np.sin(ang)], 1).astype(np.float32)).to(DEV)
        width = (H + 2 * Hk) * d
        qkv0 = gen(T, width, seed=rot, dtype=dtype)
        qkv = qkv0.clone().to(DEV)
        pos_list = [40, 41, 42, 3, 4, 17]
        seg_list = [0, 0, 0, 1, 1, 2]
        pos = torch.tensor(pos_list, dtype=torch.int32, device=DEV)
        seg = torch.tensor(seg_list, dtype=torch.int32, device=DEV)
        bt = torch.tensor([[3, 9, 1, 0, 7, 2], [5, 8, 8, 8, 8, 8], [11, 12, 4, 8, 8, 8]], dtype=torch.int32, device=DEV)
        cache = torch.zeros(13, 2, Hk, P_, d, dtype=dtype, device=DEV)
        o.rope_kv_write(qkv, 0, H * d, (H + Hk) * d, H, Hk, d, rot, table, pos, seg, bt, cache, P_)
        x = f64(qkv0)
        q = x[:, : H * d].reshape(T, H, d)
        k = x[:, H * d: (H + Hk) * d].reshape(T, Hk, d)
        v = x[:, (H + Hk) * d:].reshape(T, Hk, d)
        def rotate(z):
            r = P.rope_neox(z[..., :rot], pos_list, inv)
            return np.concatenate([r, z[..., rot:]], -1)
        tol = dict(atol=1e-6, rtol=1e-6) if dtype == torch.float32 else dict(atol=1e-6, rtol=2.0 ** -8)
        close(f64(qkv)[:, : H * d].reshape(T, H, d), rotate(q), **tol)
        assert torch.equal(qkv[:, (H + Hk) * d:].cpu(), qkv0[:, (H + Hk) * d:])  # v untouched in place
        rk = rotate(k)
        btc = bt.cpu().numpy()
        written = torch.zeros(13, P_, dtype=torch.bool)
        for t in range(T):
            page, slot = btc[seg_list[t], pos_list[t] // P_], pos_list[t] % P_
            close(f64(cache[page, 0, :, slot]), rk[t], **tol)
            close(f64(cache[page, 1].reshape(Hk, d, P_)[:, :, slot]), v[t], atol=0, rtol=0)
            written[page, slot] = True
        c = cache.cpu()
        keys_untouched = c[:, 0][~written.unsqueeze(1).expand(13, Hk, P_)]
        vals_untouched = c[:, 1].reshape(13, Hk, d, P_).permute(0, 1, 3, 2)[~written.unsqueeze(1).expand(13, Hk, P_)]
        assert keys_untouched.abs().max().item() == 0.0 and vals_untouched.abs().max().item() == 0.0


def test_argmax_rows():
    o = ops()
    lg = gen(6, 1003, seed=4).to(DEV)
    lg[1, 500] = 9.0
    lg[1, 20] = 9.0          # a tie: the first maximum wins (crates/allpaca-core/src/sampling.rs:215-225)
    lg[2, :] = float("-inf")
    lg[3, 7] = float("nan")
    lg[4, 1002] = float("inf")
    out = torch.empty(6, dtype=torch.int32, device=DEV)
    o.argmax_rows(lg, out)
    want = [P.argmax(row) for row in lg.cpu().numpy()]
    assert out.cpu().tolist() == want
    assert want[1] == 20 and want[2] == 0 and want[4] == 1002


@pytest.mark.parametrize("one_block", [False, True], ids=["many blocks a row", "one block a row"])
def test_sample_rows_against_plain_sampler(one_block):
    o = ops()
    rng = np.random.default_rng(0)
    for V in (50, 1003, 5000):
        R = 40
        lg = (gen(R, V, seed=V) * 2.0)
        lg[0, 3] = lg[0, 9] = lg[0, 30] = 7.0      # ties at the top
        lg[1, :] = float("nan")                     # degenerate
        lg[2, 5] = float("-inf")
        temps = rng.choice([0.0, 0.7, 1.0, 1.5], size=R).astype(np.float32)
        ks = rng.choice([0, 1, 5, 40, 2000], size=R).astype(np.int32)
        ps = rng.choice([1.0, 0.95, 0.5, 0.1, 0.0], size=R).astype(np.float32)
        us = rng.random(R).astype(np.float32)
        us[3] = 0.0
        us[4] = 0.99999994
        out = torch.empty(R, dtype=torch.int32, device=DEV)
        o.sample_rows(lg.to(DEV), torch.from_numpy(temps).to(DEV), torch.from_numpy(ks).to(DEV),
                      torch.from_numpy(ps).to(DEV), torch.from_numpy(us).to(DEV), out, one_block=one_block)
        mismatches = _sample_mismatches(out.cpu().tolist(), lg.numpy(), temps, ks, ps, us)
        assert not mismatches, mismatches


def _sample_mismatches(got, lgn, temps, ks, ps, us):
    """Rows whose token is not the plain sampler's.  A draw that lands within rounding of a boundary between two
    candidates may fall either way: the neighbour is accepted if the plain sampler gives it for a nudged r."""
    mismatches = []
    for r in range(len(got)):
        a = (lgn[r], float(temps[r]), int(ks[r]), float(ps[r]))
        want = P.sample(*a, float(us[r]))
        if got[r] != want:
            near = {P.sample(*a, float(us[r]) + e) for e in (-2e-6, 2e-6)}
            if got[r] not in near:
                mismatches.append((r, got[r], want) + a[1:] + (float(us[r]),))
    return mismatches


@pytest.mark.parametrize("values", ["halves", "64ths", "bfloat16", "all equal", "half of them -inf"])
def test_sample_rows_among_equal_values(values):
    """Many candidates with the same value: the k-th largest, the end of the top-p prefix and the drawn candidate
    then fall inside a run of equal values, which the order breaks by id (crates/allpaca-core/src/sampling.rs:24-67:
    a stable sort by value).  The kernels with many blocks a row carry the id in the sort key; each row must give the
    plain sampler's token, the same token as one block a row, the same alone as in the batch, and the same when the
    caller's word on which cuts its rows want is wrong (such rows go the slow way)."""
    o = ops()
    rng = np.random.default_rng(5)
    for V, R in ((701, 9), (4099, 33), (20011, 12)):   # primes: no top-p of the list is a whole share of equal values
        lg = gen(R, V, seed=V + 1) * 3.0
        if values == "halves":
            lg = torch.round(lg * 2) / 2
        elif values == "64ths":
            lg = torch.round(lg * 64) / 64
        elif values == "bfloat16":
            lg = lg.bfloat16().float()
        elif values == "all equal":
            lg[:] = 0.25
        else:
            lg[:, V // 2:] = float("-inf")
        temps = rng.choice([0.3, 0.7, 1.0, 1.5], size=R).astype(np.float32)
        # (no k of the list times a p of the list is a whole number either: with equal values a prefix that ends
        # exactly on p would be decided by rounding)
        ks = rng.choice([0, 1, 7, 41, 1001, 1023, 1025, 3001], size=R).astype(np.int32)
        ps = rng.choice([1.0, 0.99, 0.95, 0.5, 0.1, 0.0, -1.0], size=R).astype(np.float32)
        us = rng.random(R).astype(np.float32)
        d = [torch.from_numpy(a).to(DEV) for a in (temps, ks, ps, us)]
        lgd = lg.to(DEV)
        outs = {}
        for name, kw in (("many blocks", {}), ("one block", {"one_block": True}),
                         ("no cut announced", {"any_top_k": False, "any_top_p": False}),
                         ("few survivors announced", {"few_after_top_k": True}),
                         ("top-k only announced", {"any_top_p": False})):
            out = torch.empty(R, dtype=torch.int32, device=DEV)
            o.sample_rows(lgd, *d, out, **kw)
            outs[name] = out.cpu().tolist()
        mismatches = _sample_mismatches(outs["many blocks"], lg.numpy(), temps, ks, ps, us)
        assert not mismatches, (V, mismatches)
        for name, got in outs.items():
            assert got == outs["many blocks"], (V, name, got, outs["many blocks"])
        alone = torch.empty(R, dtype=torch.int32, device=DEV)
        for r in range(R):
            o.sample_rows(lgd[r:r + 1], *(t[r:r + 1] for t in d), alone[r:r + 1])
        assert alone.cpu().tolist() == outs["many blocks"], V


@pytest.mark.parametrize("one_block", [False, True], ids=["many blocks a row", "one block a row"])
def test_sample_rows_on_the_boundaries_between_candidates(one_block):
    """Rows with more than 1,024 survivors (no cut, a wide top-k, top-p alone): the many-block kernels add integer
    weights (exp in units of 2^-40), the one-block kernel walks in float32 as the reference does
    (crates/allpaca-core/src/sampling.rs:55-67) and the plain sampler in float64, so a uniform number on the boundary
    between two candidates may fall on either side.  The number is put on boundaries of the plain sampler's walk and
    one float32 step to either side: the token is the plain sampler's or its neighbour in the walk, never a
    candidate further away, on either way through the kernels; and away from the boundaries (the other sampler
    tests) it is the plain sampler's."""
    o = ops()
    V = 5000
    base = (gen(1, V, seed=77) * 2.5)[0]
    cases, rows, temps, ks, ps, us = [], [], [], [], [], []
    for temperature, top_k, top_p in ((1.0, 0, 1.0), (0.7, 2000, 1.0), (1.0, 0, 0.95), (1.3, 3000, 0.9)):
        cand, draws = P.sample_candidates(base.numpy(), temperature, top_k, top_p)
        assert draws and len(cand) > 1024
        place = {i: n for n, (i, _) in enumerate(cand)}
        edges = np.cumsum([p for _, p in cand])
        for j in np.linspace(0, len(cand) - 2, 25).astype(int):
            on = np.float32(edges[j])
            for u in (np.nextafter(on, np.float32(0)), on, np.nextafter(on, np.float32(1))):
                if 0.0 <= u < 1.0:
                    cases.append((place, P.sample(base.numpy(), temperature, top_k, top_p, float(u))))
                    rows.append(base)
                    temps.append(temperature)
                    ks.append(top_k)
                    ps.append(top_p)
                    us.append(u)
    R = len(rows)
    out = torch.empty(R, dtype=torch.int32, device=DEV)
    o.sample_rows(torch.stack(rows).to(DEV), torch.tensor(temps, device=DEV), torch.tensor(ks, dtype=torch.int32, device=DEV),
                  torch.tensor(ps, device=DEV), torch.tensor(np.asarray(us, np.float32), device=DEV), out,
                  one_block=one_block)
    got = out.cpu().tolist()
    far = [(r, got[r], want) for r, (place, want) in enumerate(cases)
           if got[r] not in place or abs(place[got[r]] - place[want]) > 1]
    assert not far, far[:5]
    assert sum(got[r] == want for r, (_, want) in enumerate(cases)) > R // 2


def test_sample_rows_frequencies():
    o = ops()
    V, n = 12, 4000
    lg = torch.tensor([0.0, 1.0, 2.0, -1.0, 0.5, 0.5, -3.0, 1.5, 0.2, -0.2, 0.9, 0.1]).repeat(n, 1).to(DEV)
    T = 0.8
    us = torch.from_numpy(np.random.default_rng(1).random(n).astype(np.float32)).to(DEV)
    out = torch.empty(n, dtype=torch.int32, device=DEV)
    o.sample_rows(lg, torch.full((n,), T, device=DEV), torch.zeros(n, dtype=torch.int32, device=DEV),
                  torch.ones(n, device=DEV), us, out)
    counts = np.bincount(out.cpu().numpy(), minlength=V)
    p = np.exp(lg[0].cpu().numpy().astype(np.float64) / T)
    p /= p.sum()
    chi2 = ((counts - n * p) ** 2 / (n * p)).sum()
    assert chi2 < 31.26  # 11 degrees of freedom, p = 0.001
