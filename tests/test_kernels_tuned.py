"""Each bfloat16 MFMA kernel alone against a float64 reference of the same operation on the same
bfloat16 inputs, at sizes other than the engine's: widths and row counts that are no multiple of a
tile, every head size in steps of 16, head counts and groups of any kind, windows, page sizes."""
import math
from types import SimpleNamespace

import numpy as np
import pytest
import torch

import plain_llama as P
from test_kernels_plain import DEV, f64, gen, make_cache

pytestmark = pytest.mark.gpu

BF = torch.bfloat16


def tuned():
    from allpaca_amd.kernels import tuned as t
    return t


def pack(w):
    from allpaca_amd.kernels.packing import pack_mfma
    return pack_mfma(w)


def test_packing_roundtrip_and_lane_order():
    from allpaca_amd.kernels.packing import pack_mfma, unpack_mfma
    w = gen(50, 72, seed=1, dtype=BF)
    p = pack_mfma(w)
    assert tuple(p.data.shape) == (4, 3, 64, 8) and torch.equal(unpack_mfma(p), w)
    i, c = 5, 3          # lane c*16 + i of tile (band 1, chunk 2) holds w[16 + i, 64 + 8c : 64 + 8c + 8]
    wide = torch.zeros(64, 96, dtype=BF)
    wide[:50, :72] = w
    assert torch.equal(p.data[1, 2, c * 16 + i], wide[16 + i, 64 + c * 8: 64 + c * 8 + 8])


def check(got, want, out_dtype):
    """Sums are float32 over exact bfloat16 products: the result is within float32 summation error of the
    float64 value, plus one rounding to bfloat16 if it is stored so."""
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    scale = np.abs(want).max() + 1e-30
    d = np.abs(got - want)
    tol = 1e-5 * scale + (2.0 ** -8) * np.abs(want) if out_dtype == BF else 1e-5 * scale + 1e-5 * np.abs(want)
    assert (d <= tol).all(), f"max diff {d.max():.3e} (scale {scale:.3e}) at {np.unravel_index((d - tol).argmax(), d.shape)}"


# rows 17..128 with a long K go through the kernel that cuts K into slices (the last slice may be shorter or empty)
GEMM_SHAPES = [(1, 5, 16), (3, 100, 136), (8, 4096, 512), (16, 33, 1208), (17, 257, 72), (33, 64, 8), (64, 130, 264),
               (65, 64, 64), (128, 129, 72), (200, 300, 200), (300, 515, 120), (1000, 40, 1024),
               (40, 200, 1208), (64, 130, 2056), (100, 96, 520), (128, 48, 4096), (130, 200, 320), (256, 130, 192),
               # enough blocks for the 256-row tiles: a last tile of 232 rows, K a multiple of 64 and not
               (1000, 8192, 200), (1024, 8190, 192),
               # 129..1024 rows and few output columns: K in slices (5, 2 and 3 of them), a last row tile of 44 rows
               (512, 384, 2048), (200, 4096, 520), (300, 1100, 1024),
               # 1,024 rows or more, K a multiple of 128, N of 4: the kernel whose weights go straight into registers.
               # One and several passes of its loop over K; a last row tile of 76 and of 6 rows; a last band of 4
               # columns; 4, 6 and 8 bands a wave (6,144 and 8,192 columns at 2,048 rows)
               (1024, 256, 128), (1100, 1028, 384), (1030, 2500, 640), (2048, 6144, 128), (2048, 8192, 256),
               (2048, 4096, 1024),
               (2048, 10240, 128), (1100, 16384, 256),
               # 3 and 5 bands a wave: the widths of a 3B model (3,072 and 5,120 columns)
               (2048, 3072, 128), (2048, 5120, 256),
               # few output columns and a long K: K in two slices on that kernel, then the kernel that adds them
               (2048, 1024, 8192), (1100, 512, 4096)]


@pytest.mark.parametrize("M,N,K", GEMM_SHAPES)
def test_gemm_bf16(M, N, K):
    t = tuned()
    a, w = gen(M, K, seed=1, dtype=BF).to(DEV), gen(N, K, seed=2, dtype=BF).to(DEV)
    want = f64(a) @ f64(w).T
    wp = pack(w)
    for out_dtype in (BF, torch.float32):
        out = torch.full((M, N), 7.0, dtype=out_dtype, device=DEV)
        t.gemm_bf16(a, wp, out)
        check(f64(out), want, out_dtype)
    acc = gen(M, N, seed=3).to(DEV)
    before = f64(acc)
    t.gemm_bf16(a, wp, acc, accumulate=True)
    check(f64(acc) - before, want, torch.float32)


def test_gemm_bf16_strided_views_and_padding_rows_untouched():
    t = tuned()
    big = gen(40, 200, seed=5, dtype=BF).to(DEV)
    a = big[:, 16:16 + 72]                              # row stride 200, offset 32 bytes
    w = gen(50, 72, seed=6, dtype=BF).to(DEV)
    wide = torch.full((40, 64), 3.0, dtype=BF, device=DEV)
    out = wide[:, 8:58]                                 # out is a view too: columns beside it must stay
    t.gemm_bf16(a, pack(w), out)
    check(f64(out), f64(a) @ f64(w).T, BF)
    assert (wide[:, :8] == 3.0).all() and (wide[:, 58:] == 3.0).all()


def test_widths_the_mfma_kernels_do_not_take_stay_row_major_and_run_on_the_plain_kernel():
    from allpaca_amd.kernels import ops
    a, w = gen(5, 13, seed=1, dtype=BF).to(DEV), gen(7, 13, seed=2, dtype=BF).to(DEV)   # K = 13
    kept = ops.prepare_matrix(w, BF)
    assert isinstance(kept, torch.Tensor)                   # no tiled form for this width
    assert not isinstance(ops.prepare_matrix(gen(7, 16, dtype=BF).to(DEV), BF), torch.Tensor)
    assert isinstance(ops.prepare_matrix(gen(7, 16).to(DEV), torch.float32), torch.Tensor)
    out = torch.empty(5, 7, dtype=BF, device=DEV)
    ops.linear(a, kept, out)
    check(f64(out), f64(a) @ f64(w).T, BF)


def test_skinny_rows_together_equal_each_row_alone():
    """A decoded row is the same alone and in any batch of up to 16 rows, bit for bit."""
    t = tuned()
    for N, K in [(4096, 512), (100, 1208), (33, 72)]:
        a, w = gen(16, K, seed=3, dtype=BF).to(DEV), pack(gen(N, K, seed=4, dtype=BF).to(DEV))
        tog = torch.empty(16, N, dtype=torch.float32, device=DEV)
        t.gemm_bf16(a, w, tog)
        for r in (0, 7, 15):
            alone = torch.empty(1, N, dtype=torch.float32, device=DEV)
            t.gemm_bf16(a[r:r + 1], w, alone)
            assert torch.equal(alone[0], tog[r])
        some = torch.empty(5, N, dtype=torch.float32, device=DEV)
        t.gemm_bf16(a[3:8], w, some)
        assert torch.equal(some, tog[3:8])


def bf16_round(a):
    """float64 array rounded to bfloat16 (nearest even), as float64."""
    return f64(torch.from_numpy(np.asarray(a, np.float32)).to(BF))


def emit_reference(a, w, res, g):
    """What the emitting product leaves: the new residual, the row bfloat16(residual * g), sums of squares."""
    x = res + f64(a) @ f64(w).T
    return x, bf16_round(x * f64(g)), (x ** 2).sum(axis=1, keepdims=True)


@pytest.mark.parametrize("M,D,K", [(1, 64, 32), (8, 4096, 512), (16, 104, 1208), (5, 40, 72), (3, 8192, 264)])
def test_product_into_the_residual_leaves_the_next_norms_row(M, D, K):
    """residual += a . w^T; raw = bfloat16(residual * g); ss[band][row] = sum of residual^2 over the band."""
    t = tuned()
    a, w = gen(M, K, seed=1, dtype=BF).to(DEV), gen(D, K, seed=2, dtype=BF).to(DEV)
    res = gen(M, D, seed=3, scale=2.0).to(DEV)
    res[0] *= 30.0
    g = (1 + 0.2 * gen(D, seed=4)).to(DEV)
    x, raw_want, ss_want = emit_reference(a, w, f64(res), g)
    left = t.gemm_emit_bf16(a, pack(w), res, g)
    assert left is not None
    raw, ss = left
    check(f64(res), x, torch.float32)
    bands = -(-D // 16)
    assert tuple(ss.shape) == (16, -(-bands // 4) * 4) and tuple(raw.shape) == (M, D)
    assert np.allclose(f64(ss)[:M, :bands].sum(axis=1), ss_want[:, 0], rtol=1e-5)
    band = f64(ss)[:M, 1] if D >= 32 else None
    if band is not None:
        assert np.allclose(band, (x[:, 16:32] ** 2).sum(axis=1), rtol=1e-5, atol=1e-6)
    # x carries the float32 noise of its sum (as `check` allows for it); on top of that one rounding to bfloat16
    d = np.abs(f64(raw) - raw_want)
    assert (d <= 2.0 ** -7 * np.abs(raw_want) + 1.5e-5 * np.abs(x).max()).all() and (d > 0).mean() < 0.01


@pytest.mark.parametrize("M,N,K", [(1, 40, 64), (8, 4096, 512), (16, 100, 1200), (5, 34, 72), (2, 36, 104), (3, 6144, 4096),
                                   (16, 2050 * 16, 136), (7, 48, 8192)])
def test_product_of_the_normalised_row_from_what_was_left(M, N, K):
    """out = (raw . W^T) / sqrt(sum(ss) / K + eps), which is rmsnorm(x) . W^T up to the rounding of x * g."""
    t = tuned()
    x = f64(gen(M, K, seed=1, scale=3.0))
    x[0, : K // 2] *= 40.0                               # rows of very different size: one root per row
    g = f64(1 + 0.2 * gen(K, seed=2))
    w = gen(N, K, seed=3, dtype=BF).to(DEV)
    eps = 3e-4
    raw64 = bf16_round(x * g)
    raw = torch.from_numpy(raw64).to(BF).to(DEV)
    bands = -(-K // 16)
    xp = np.zeros((M, bands * 16)); xp[:, :K] = x
    ss64 = np.full((16, -(-bands // 4) * 4), 1e30); ss64[:M, :bands] = (xp.reshape(M, bands, 16) ** 2).sum(axis=2)
    ss64[M:, :bands] = 0.0                              # beyond the bands: never read, whatever it holds
    ss = torch.from_numpy(ss64).float().to(DEV)
    rstd = 1.0 / np.sqrt((x ** 2).mean(axis=1, keepdims=True) + eps)
    want = (raw64 @ f64(w).T) * rstd
    for out_dtype in (BF, torch.float32):
        out = torch.full((M, N), 7.0, dtype=out_dtype, device=DEV)
        assert t.gemm_pre_bf16(raw, ss, eps, pack(w), out)
        check(f64(out), want, out_dtype)
    exact = (x * rstd * g) @ f64(w).T
    assert np.abs(f64(out) - exact).max() <= 2.0 ** -8 * np.abs(x * rstd * g).max() * np.abs(f64(w)).sum(axis=1).max()


@pytest.mark.parametrize("M,F,K", [(1, 24, 64), (8, 176, 512), (16, 200, 112), (4, 14336 // 8, 1024), (8, 14336, 512),
                                   (11, 9000, 256)])
def test_swiglu_of_the_normalised_row_from_what_was_left(M, F, K):
    t = tuned()
    x = f64(gen(M, K, seed=1, scale=2.0))
    g = f64(1 + 0.2 * gen(K, seed=2))
    w = gen(2 * F, K, seed=3, scale=0.3, dtype=BF).to(DEV)
    eps = 1e-5
    raw64 = bf16_round(x * g)
    bands = -(-K // 16)
    ss64 = np.zeros((16, -(-bands // 4) * 4)); ss64[:M, :bands] = (x.reshape(M, bands, 16) ** 2).sum(axis=2)
    rstd = 1.0 / np.sqrt((x ** 2).mean(axis=1, keepdims=True) + eps)
    out = torch.empty(M, F, dtype=BF, device=DEV)
    assert t.swiglu_pre_bf16(torch.from_numpy(raw64).to(BF).to(DEV), torch.from_numpy(ss64).float().to(DEV), eps,
                             pack(w[:F].contiguous()), pack(w[F:].contiguous()), out)
    check(f64(out), P.silu(raw64 @ f64(w[:F]).T * rstd) * (raw64 @ f64(w[F:]).T * rstd), BF)


@pytest.mark.parametrize("M,D,K", [(40, 520, 1208), (64, 4096, 512), (100, 300, 2056), (17, 256, 520), (300, 520, 1208),
                                   (1000, 264, 1024)])
def test_product_into_the_residual_leaves_the_next_norms_row_with_more_than_16_rows(M, D, K):
    """The same from the tiled kernel with K in slices: the finishing kernel leaves sums of squares per row and block
    of 256 columns."""
    t = tuned()
    a, w = gen(M, K, seed=1, dtype=BF).to(DEV), gen(D, K, seed=2, dtype=BF).to(DEV)
    res = gen(M, D, seed=3, scale=2.0).to(DEV)
    res[0] *= 30.0
    g = (1 + 0.2 * gen(D, seed=4)).to(DEV)
    x, raw_want, ss_want = emit_reference(a, w, f64(res), g)
    left = t.gemm_emit_bf16(a, pack(w), res, g)
    assert left is not None
    raw, ss = left
    check(f64(res), x, torch.float32)
    width = 256
    parts = -(-D // width)
    assert tuple(ss.shape) == (M, parts) and tuple(raw.shape) == (M, D)
    xp = np.zeros((M, parts * width)); xp[:, :D] = x
    assert np.allclose(f64(ss), (xp.reshape(M, parts, width) ** 2).sum(axis=2), rtol=1e-5, atol=1e-6)
    # x carries the float32 noise of its sum (as `check` allows for it); on top of that one rounding to bfloat16
    d = np.abs(f64(raw) - raw_want)
    assert (d <= 2.0 ** -7 * np.abs(raw_want) + 1.5e-5 * np.abs(x).max()).all() and (d > 0).mean() < 0.01
    if D % 8:
        return       # a width the MFMA products do not take as their K: the norm's own kernel runs instead
    # and the product behind the norm takes what was left
    N2 = 72
    w2 = gen(N2, D, seed=5, dtype=BF).to(DEV)
    eps = 1e-5
    out = torch.empty(M, N2, dtype=BF, device=DEV)
    assert t.gemm_pre_bf16(raw, ss, eps, pack(w2), out)
    rstd = 1.0 / np.sqrt((x ** 2).mean(axis=1, keepdims=True) + eps)
    check(f64(out), (f64(raw) @ f64(w2).T) * rstd, BF)


@pytest.mark.parametrize("M,D,K,slices", [
    # K in one piece: a part per tile of columns (tiles of 3 to 8 bands a wave; many columns in two launches, whole
    # rounds of wide tiles and the rest), a last row tile of 76 and of 6 rows, columns that end inside a tile
    (1100, 520, 1280, 1), (1030, 4096, 256, 1), (1100, 15000, 128, 1), (2048, 1028, 384, 1), (2048, 14336, 128, 1),
    # K in two slices: a part per 1,024 columns
    (1100, 1024, 4096, 2), (1030, 2500, 4608, 2)])
def test_product_into_the_residual_leaves_the_next_norms_row_with_more_than_1024_rows(M, D, K, slices):
    """From the product that loads its weights straight into registers: its epilogue adds into the residual, writes the
    row times the next norm's weight and the rows' sums of squares over its tile of columns; with K in two slices the
    kernel that adds the slices does.  Then the products behind the norm take what was left: one that stores, and
    SwiGLU."""
    t = tuned()
    a, w = gen(M, K, seed=1, dtype=BF).to(DEV), gen(D, K, seed=2, dtype=BF).to(DEV)
    res = gen(M, D, seed=3, scale=2.0).to(DEV)
    res[0] *= 30.0
    g = (1 + 0.2 * gen(D, seed=4)).to(DEV)
    x, raw_want, ss_want = emit_reference(a, w, f64(res), g)
    left = t.gemm_emit_bf16(a, pack(w), res, g)
    assert left is not None
    raw, ss = left
    check(f64(res), x, torch.float32)
    from allpaca_amd.kernels import lib
    assert lib.load("tuned").apc_gemm_direct_k_split(M, D, K) == slices
    assert ss.shape[0] == M and 1 <= ss.shape[1] <= 256 and tuple(raw.shape) == (M, D)
    if slices > 1:
        assert ss.shape[1] == -(-D // 1024)
    assert np.allclose(f64(ss).sum(axis=1), (x ** 2).sum(axis=1), rtol=1e-5)
    d = np.abs(f64(raw) - raw_want)
    assert (d <= 2.0 ** -7 * np.abs(raw_want) + 1.5e-5 * np.abs(x).max()).all() and (d > 0).mean() < 0.01
    if D % 128:
        return       # no K for the product with the weights in registers
    eps = 1e-5
    rstd = 1.0 / np.sqrt((x ** 2).mean(axis=1, keepdims=True) + eps)
    N2 = 264
    w2 = gen(N2, D, seed=5, dtype=BF).to(DEV)
    out = torch.empty(M, N2, dtype=BF, device=DEV)
    assert t.gemm_pre_bf16(raw, ss, eps, pack(w2), out)
    check(f64(out), (f64(raw) @ f64(w2).T) * rstd, BF)
    F = 136
    w3 = gen(2 * F, D, seed=6, dtype=BF).to(DEV)
    out = torch.empty(M, F, dtype=BF, device=DEV)
    assert t.swiglu_pre_bf16(raw, ss, eps, pack(w3[:F].contiguous()), pack(w3[F:].contiguous()), out)
    check(f64(out), P.silu(f64(raw) @ f64(w3[:F]).T * rstd) * (f64(raw) @ f64(w3[F:]).T * rstd), BF)


@pytest.mark.parametrize("M,N,K", [(40, 200, 1208), (64, 6144, 4096), (100, 96, 520), (128, 130, 2048),
                                   # K in one piece (enough tiles without slices): 224 and 192 tiles; a last row tile of 44
                                   (64, 28672, 520), (300, 8192, 264), (300, 2048, 1288),
                                   # SwiGLU on the 256-row tile with the norm's scale in its epilogue
                                   (1024, 2 * 16640, 128),
                                   # SwiGLU from 384 rows on: the kernel that loads its weights straight into registers,
                                   # the norm's scale in its epilogue (a last row tile of 116, of 128 and of 0 rows)
                                   (500, 2 * 1200, 384), (384, 2 * 264, 128), (640, 2 * 2056, 256)])
def test_product_of_the_normalised_row_from_what_was_left_with_17_to_1024_rows(M, N, K):
    """On the tiled kernel, with K in slices (the finishing kernel scales) or whole (the product's epilogue does)."""
    t = tuned()
    whole = t._tiled_k_split(M, N, K) == 1
    assert whole == ((M, N, K) in [(64, 28672, 520), (300, 8192, 264), (1024, 2 * 16640, 128), (500, 2 * 1200, 384),
                                   (384, 2 * 264, 128), (640, 2 * 2056, 256)])
    x = f64(gen(M, K, seed=1, scale=3.0))
    x[0, : K // 2] *= 40.0
    g = f64(1 + 0.2 * gen(K, seed=2))
    w = gen(N, K, seed=3, dtype=BF).to(DEV)
    eps = 3e-4
    raw64 = bf16_round(x * g)
    raw = torch.from_numpy(raw64).to(BF).to(DEV)
    parts = -(-K // 256)
    xp = np.zeros((M, parts * 256)); xp[:, :K] = x
    ss = torch.from_numpy((xp.reshape(M, parts, 256) ** 2).sum(axis=2)).float().contiguous().to(DEV)
    rstd = 1.0 / np.sqrt((x ** 2).mean(axis=1, keepdims=True) + eps)
    want = (raw64 @ f64(w).T) * rstd
    for out_dtype in (BF, torch.float32):
        out = torch.full((M, N), 7.0, dtype=out_dtype, device=DEV)
        assert t.gemm_pre_bf16(raw, ss, eps, pack(w), out)
        check(f64(out), want, out_dtype)
    F = N // 2 // 8 * 8                                  # and SwiGLU on the same row
    if F:
        out = torch.empty(M, F, dtype=BF, device=DEV)
        assert t.swiglu_pre_bf16(raw, ss, eps, pack(w[:F].contiguous()), pack(w[F:2 * F].contiguous()), out)
        check(f64(out), P.silu(raw64 @ f64(w[:F]).T * rstd) * (raw64 @ f64(w[F:2 * F]).T * rstd), BF)


def test_folded_norm_refuses_what_it_does_not_take():
    t = tuned()
    w = pack(gen(32, 64, dtype=BF).to(DEV))
    g = torch.ones(32, device=DEV)
    assert t.gemm_emit_bf16(gen(17, 64, dtype=BF).to(DEV), w, torch.zeros(17, 32, device=DEV), g) is None   # short K
    assert t.gemm_emit_bf16(gen(1100, 64, dtype=BF).to(DEV), w, torch.zeros(1100, 32, device=DEV), g) is None
    assert t.gemm_emit_bf16(gen(17, 64, dtype=BF).to(DEV), w, torch.zeros(17, 32, device=DEV), g[:31]) is None   # g
    ss = torch.zeros(16, 4, device=DEV)
    out = torch.empty(17, 32, dtype=BF, device=DEV)
    assert not t.gemm_pre_bf16(gen(17, 64, dtype=BF).to(DEV), ss, 1e-5, w, out)
    assert not t.gemm_pre_bf16(gen(4, 64, dtype=BF).to(DEV), ss[:, :3], 1e-5, w, out[:4])                   # ss too short


def test_embedding_from_the_tiled_table():
    from allpaca_amd.kernels import ops
    table = gen(515, 120, seed=1, dtype=BF).to(DEV)
    toks = torch.tensor([0, 514, 17, 16, 15, 17], dtype=torch.int32, device=DEV)
    out = torch.empty(6, 120, device=DEV)
    ops.embed_rows(pack(table), toks, out)
    assert torch.equal(out.cpu(), table.float().cpu()[toks.cpu().long()])


@pytest.mark.parametrize("M,F,K", [(1, 24, 64), (8, 176, 64), (9, 200, 120), (64, 512, 192), (65, 40, 72), (300, 520, 1024),
                                   (130, 200, 120), (300, 512, 192), (256, 14336 // 8, 512), (48, 176, 1032),
                                   (100, 72, 2048), (300, 200, 320), (1000, 4096, 200), (1024, 4090, 128),
                                   # the 256-row tile (1,024 rows or more, K a multiple of 64, 512 tiles or more): last
                                   # row tile of 76 rows, last column tile of 16 columns; one and three K steps
                                   (2048, 8192, 128), (1100, 13200, 192), (1024, 16640, 64),
                                   # weights straight into registers (K a multiple of 128): 2, 3 and 4 gate bands a
                                   # wave, a last band of 8 columns, a last row tile of 76 rows
                                   (1024, 136, 128), (1100, 13208, 256), (2048, 3072, 384), (2048, 14336 // 2, 128),
                                   (2048, 14336, 128),
                                   # few rows and more than 512 bands of outputs: two gate bands and their up bands a
                                   # block of the streaming kernel (an odd number of bands; a last band of 8 columns)
                                   (8, 14336, 256), (16, 9000, 64), (3, 8200, 520)])
def test_swiglu_bf16(M, F, K):
    t = tuned()
    h = gen(M, K, seed=1, dtype=BF).to(DEV)
    w = gen(2 * F, K, seed=2, scale=0.3, dtype=BF).to(DEV)
    out = torch.empty(M, F, dtype=BF, device=DEV)
    t.swiglu_bf16(h, pack(w[:F].contiguous()), pack(w[F:].contiguous()), out)
    g = f64(h) @ f64(w[:F]).T
    u = f64(h) @ f64(w[F:]).T
    check(f64(out), P.silu(g) * u, BF)


@pytest.mark.parametrize("H,Hk,d,rot,P_,with_cache", [(32, 8, 128, 128, 16, True), (5, 1, 64, 32, 8, True),
                                                      (6, 2, 80, 0, 16, True), (4, 4, 256, 256, 32, False),
                                                      (3, 3, 48, 48, 24, True),
                                                      # pages whose columns do not start on 16 bytes: values slot by slot
                                                      (4, 2, 64, 64, 12, True),
                                                      # more columns of values than a block has in LDS at a time
                                                      (8, 8, 128, 128, 16, True)])
def test_rotation_and_cache_write_16_bytes_a_lane_equals_the_plain_kernel(H, Hk, d, rot, P_, with_cache):
    """`ops.rope_kv_write` on bfloat16 rows takes the kernel of the MFMA library; the plain kernel on the same input
    gives the same rows and the same cache (the same float32 formula; a rounding may fall the other way where the
    compiler fused a multiply and an add differently: few elements, one unit of bfloat16)."""
    from allpaca_amd.kernels import lib, ops
    T = 70
    rng = np.random.default_rng(d + rot)
    lens = [33, 20, 17]                                 # three segments: rows are their last positions
    pos_list = [p for n, first in zip(lens, (40, 0, 100)) for p in range(first, first + n)]
    seg_list = [s_ for s_, n in enumerate(lens) for _ in range(n)]
    pos = torch.tensor(pos_list, dtype=torch.int32, device=DEV)
    seg = torch.tensor(seg_list, dtype=torch.int32, device=DEV)
    max_blocks = -(-140 // P_)
    bt = torch.from_numpy(rng.permutation(3 * max_blocks).reshape(3, max_blocks).astype(np.int32)).to(DEV)
    width = (H + 2 * Hk) * d + 8
    qkv0 = gen(T, width, seed=1, dtype=BF).to(DEV)
    ang = np.arange(140)[:, None] * (1.0 / 300.0 ** (np.arange(rot // 2) / max(rot // 2, 1)))[None, :]
    table = torch.from_numpy(np.stack([np.cos(ang), np.sin(ang)], 1).astype(np.float32)).to(DEV) if rot else None
    offs = (8, 8 + H * d, 8 + (H + Hk) * d)
    results = []
    for which in ("tuned", "plain"):
        qkv = qkv0.clone()
        cache = torch.zeros(3 * max_blocks, 2, Hk, P_, d, dtype=BF, device=DEV) if with_cache else None
        if which == "tuned":
            ops.rope_kv_write(qkv, *offs, H, Hk, d, rot, table, pos, seg, bt, cache, P_)
        else:
            lib.check(lib.load("plain").apc_rope_kv_write(
                qkv.data_ptr(), 1, width, *offs, T, H, Hk, d, rot, table.data_ptr() if rot else 0, pos.data_ptr(),
                seg.data_ptr(), bt.data_ptr(), max_blocks, cache.data_ptr() if with_cache else 0, 1, P_,
                torch.cuda.current_stream().cuda_stream), "rope")
        results.append((f64(qkv), f64(cache) if with_cache else np.zeros(1)))
    for a, b in zip(results[0], results[1]):
        diff = np.abs(a - b)
        assert (diff <= 2.0 ** -7 * np.abs(b) + 1e-30).all() and (diff > 0).mean() < 0.005
    assert np.array_equal(results[0][0][:, :8], f64(qkv0)[:, :8])              # columns beside the heads stay
    if with_cache:
        assert (results[0][1] != 0).any()


@pytest.mark.parametrize("M,H,Hk,d,K,P_,pre", [(8, 32, 8, 128, 4096, 16, True), (5, 6, 2, 64, 328, 8, True),
                                               (16, 3, 3, 32, 72, 24, False), (1, 5, 1, 96, 200, 16, True),
                                               (3, 4, 2, 256, 264, 32, False),
                                               # more than 16 rows: in the finishing kernel of the product with K in slices
                                               (17, 6, 2, 64, 520, 8, True), (64, 32, 8, 128, 4096, 16, True),
                                               (100, 3, 1, 32, 1032, 16, False), (300, 4, 2, 256, 2048, 32, True)])
def test_product_for_q_k_v_that_rotates_and_fills_the_pages_equals_the_kernels_one_after_the_other(M, H, Hk, d, K, P_, pre):
    """One kernel for q, k, v, the rotation and the cache write (the streaming kernel up to 16 rows, the finishing
    kernel of the tiled product with K in slices beyond) gives what the product followed by `rope_kv_write` gives:
    the same rotated q, the same pages (sums rounded to bfloat16 before the rotation in both)."""
    from allpaca_amd.kernels import ops
    t = tuned()
    rng = np.random.default_rng(M * 1000 + d)
    N = (H + 2 * Hk) * d
    w = pack(gen(N, K, seed=3, dtype=BF).to(DEV))
    a = gen(M, K, seed=1, dtype=BF, scale=2.0).to(DEV)
    eps = 2e-5
    ss = None
    if pre and M <= 16:
        bands = -(-K // 16)
        ss = torch.zeros(16, -(-bands // 4) * 4, device=DEV)
        ss[:M, :bands] = torch.from_numpy(rng.uniform(0.5, 40.0, (M, bands)).astype(np.float32)).to(DEV)
    elif pre:
        ss = torch.from_numpy(rng.uniform(0.5, 40.0, (M, -(-K // 256))).astype(np.float32)).to(DEV)
    max_blocks = max(5, -(-M // P_) + 2)
    max_pos = max_blocks * P_
    # rows of three segments at scattered places of the cache (no two on one), among them a page's last and first slot
    forced = [(0, P_ - 1), (1, 2 * P_)][:M]
    others = [(int(v) // max_pos, int(v) % max_pos) for v in rng.permutation(3 * max_pos)]
    places = forced + [pl for pl in others if pl not in forced][:M - len(forced)]
    seg_list, pos_list = [pl[0] for pl in places], [pl[1] for pl in places]
    pos = torch.tensor(pos_list, dtype=torch.int32, device=DEV)
    seg = torch.tensor(seg_list, dtype=torch.int32, device=DEV)
    bt = torch.from_numpy(rng.permutation(3 * max_blocks).reshape(3, max_blocks).astype(np.int32)).to(DEV)
    ang = np.arange(max_pos)[:, None] * (1.0 / 300.0 ** (np.arange(d // 2) / (d // 2)))[None, :]
    table = torch.from_numpy(np.stack([np.cos(ang), np.sin(ang)], 1).astype(np.float32)).to(DEV)
    results = []
    for fused in (True, False):
        qkv = torch.full((M, N), 3.0, dtype=BF, device=DEV)
        cache = torch.zeros(3 * max_blocks, 2, Hk, P_, d, dtype=BF, device=DEV)
        if fused:
            assert ops.qkv_rope_write(a, (ss, eps) if pre else None, w, qkv, H, Hk, d, table, pos, seg, bt, cache, P_)
        else:
            if pre:
                assert t.gemm_pre_bf16(a, ss, eps, w, qkv)
            else:
                ops.linear(a, w, qkv)
            ops.rope_kv_write(qkv, 0, H * d, (H + Hk) * d, H, Hk, d, d, table, pos, seg, bt, cache, P_)
        c64 = f64(cache)
        results.append((f64(qkv)[:, :H * d].reshape(M, H, 2, d // 2), c64[:, 0].reshape(-1, Hk, P_, 2, d // 2), c64[:, 1]))
    # The two ways add the waves' partial sums in different orders: the float32 sums differ by their summation noise
    # (1e-5 of the largest, as `check` allows; it is all there is to a sum that cancels to almost nothing), and now
    # and then a sum falls on the other side of a rounding to bfloat16: one unit of one element of a pair, which the
    # rotation spreads over the pair (its length is what the rotation keeps), and one unit of the result.
    for which, (got, want) in enumerate(zip(results[0], results[1])):
        diff = np.abs(got - want)
        pair = np.sqrt((want ** 2).sum(axis=-2, keepdims=True)) if which < 2 else 0.0
        tol = 2.0 ** -7 * np.abs(want) + 2.0 ** -7 * pair + 1e-5 * np.abs(want).max()
        assert (diff <= tol).all() and (diff > 0).mean() < 0.02
    assert (results[0][1] != 0).sum() + (results[0][2] != 0).sum() == M * 2 * Hk * d   # every row wrote its k and v, once


def test_product_for_q_k_v_that_rotates_declines_what_it_does_not_take():
    from allpaca_amd.kernels import ops
    H, Hk, d, K, P_ = 2, 1, 48, 64, 16                                          # head size no multiple of 32
    w = pack(gen((H + 2 * Hk) * d, K, seed=3, dtype=BF).to(DEV))
    table = torch.zeros(32, 2, d // 2, device=DEV)
    z = torch.zeros(4, dtype=torch.int32, device=DEV)
    bt = torch.zeros(1, 2, dtype=torch.int32, device=DEV)
    cache = torch.zeros(2, 2, Hk, P_, d, dtype=BF, device=DEV)
    qkv = torch.zeros(4, (H + 2 * Hk) * d, dtype=BF, device=DEV)
    a = gen(4, K, seed=1, dtype=BF).to(DEV)
    assert not ops.qkv_rope_write(a, None, w, qkv, H, Hk, d, table, z, z, bt, cache, P_)
    assert not cache.any() and not qkv.any()
    a17 = gen(17, K, seed=1, dtype=BF).to(DEV)                                   # more rows than the kernel takes
    w2 = pack(gen(4 * 64, K, seed=3, dtype=BF).to(DEV))
    cache2 = torch.zeros(2, 2, 1, P_, 64, dtype=BF, device=DEV)
    assert not ops.qkv_rope_write(a17, None, w2, torch.zeros(17, 256, dtype=BF, device=DEV), 2, 1, 64,
                                  torch.zeros(32, 2, 32, device=DEV), torch.zeros(17, dtype=torch.int32, device=DEV),
                                  torch.zeros(17, dtype=torch.int32, device=DEV), bt, cache2, P_)


def run_attention(H, Hk, d, P_, lens, rows_per_seg, window=0, seed=0, stale=0.0, loud=None, ranges=None, relocate=None):
    """Sequences of `lens` keys in the cache; the last `rows_per_seg[s]` positions of sequence s are the step's rows.
    `ranges`: into how many ranges the kernel for tiles of 128 rows is expected to cut the keys of this step.
    `stale`: what lies in the slots beyond a sequence's last key and in the spare page; with a window, the pages that
    every row of the step has passed are marked as given back in the block table (the spare page stands in).
    `loud`: (sequence, position, factor) of a key whose scores dwarf all others.
    `relocate`: (cache, block tables) -> the same pages at other places of another cache tensor."""
    from allpaca_amd.engine.batch import Entry, pack_step
    from allpaca_amd.kernels import ops as kernel_ops
    t = tuned()
    cache, bt, ks, vs = make_cache(lens, Hk, d, P_, BF, seed=seed, stale=stale, loud=loud)
    if relocate is not None:
        cache, bt = relocate(cache, bt)
    pos0 = [n - r for n, r in zip(lens, rows_per_seg)]
    entries = [Entry(i, [0] * r, []) for i, r in enumerate(rows_per_seg)]
    tables = [[list(bt[i, : -(-n // P_)].cpu().numpy()) for i, n in enumerate(lens)]]
    used = {int(p) for tb in tables[0] for p in tb}
    spare = next(p for p in range(cache.shape[0]) if p not in used)
    if window:
        for tb, p0 in zip(tables[0], pos0):
            for b in range(max(0, p0 - window + 1) // P_):
                tb[b] = -1
    step = pack_step(entries, pos0, [0] * len(lens), tables, torch.device(DEV), [spare],
                     tile_rows=kernel_ops.attention_tile_rows(BF))
    T = sum(rows_per_seg)
    if ranges is not None:
        assert t._key_splits(step, H, window) == ranges
    # queries scaled up: scores of deviation ~2.5, so a few keys carry each row and a wrong or missing one shows
    q = gen(T, H * d + 16, seed=seed + 7, scale=2.5, dtype=BF).to(DEV)
    out = torch.zeros(T, H * d, dtype=BF, device=DEV)
    assert t.attention_bf16(q, 16, out, H, Hk, d, cache, P_, step.block_tables[0], step, window=window)
    got = f64(out).reshape(T, H, d)
    q64 = f64(q)[:, 16:].reshape(T, H, d)
    at = 0
    for s, r in enumerate(rows_per_seg):
        want = P.attention(q64[at:at + r], f64(ks[s]), f64(vs[s]), H, Hk, window=window or None)
        d_ = np.abs(got[at:at + r] - want)
        # P and the output are rounded to bfloat16: 2^-8 of the largest value that enters a sum
        tol = 2.0 ** -7 * np.abs(f64(vs[s])).max() * 0.25 + 2.0 ** -8 * np.abs(want)
        assert (d_ <= tol).all(), (f"segment {s} rows {r}: max diff {d_.max():.3e} at "
                                   f"{np.unravel_index((d_ - tol).argmax(), d_.shape)}")
        at += r


@pytest.fixture(params=["last block merges", "merge kernel", "ranges of 64 keys from position 0", "five ranges a row"])
def decode_path(request, monkeypatch):
    """Single rows whose keys are split over blocks: the block that finishes last adds the blocks' results (the
    default), or a second kernel does; ranges of a given length for all rows instead of each row's own keys in equal
    ranges; ranges so long that a wave takes them in pieces."""
    monkeypatch.setattr(tuned(), "LAST_BLOCK_MERGES", request.param != "merge kernel")
    if request.param == "ranges of 64 keys from position 0":
        monkeypatch.setattr(tuned(), "KEYS_PER_PART", 64)
    if request.param == "five ranges a row":
        monkeypatch.setattr(tuned(), "_decode_parts", lambda pairs, span: 5)
    return request.param


@pytest.mark.parametrize("d", [16, 32, 48, 64, 80, 96, 112, 128, 160, 192, 256])
def test_attention_every_head_size(d, decode_path):
    run_attention(H=4, Hk=2, d=d, P_=16, lens=[150, 70, 33], rows_per_seg=[150, 1, 5], seed=d)


@pytest.mark.parametrize("H,Hk", [(1, 1), (3, 3), (5, 1), (6, 2), (32, 8), (20, 1), (34, 2)])
def test_attention_heads_and_groups(H, Hk, decode_path):
    # 20:1 and 17:1 groups are wider than one 16-row MFMA tile
    run_attention(H=H, Hk=Hk, d=32, P_=16, lens=[100, 260, 64], rows_per_seg=[1, 1, 64], seed=H)


@pytest.mark.parametrize("P_", [8, 16, 24, 32, 64, 128])
def test_attention_page_sizes(P_, decode_path):
    run_attention(H=4, Hk=1, d=64, P_=P_, lens=[300, 129, 64, 1], rows_per_seg=[1, 129, 2, 1], seed=P_)


@pytest.mark.parametrize("window", [1, 5, 64, 100, 1000])
def test_attention_windows(window, decode_path):
    run_attention(H=4, Hk=2, d=32, P_=16, lens=[300, 200, 90], rows_per_seg=[1, 200, 17], window=window, seed=window)


@pytest.mark.parametrize("d,window", [(192, 100), (256, 37), (128, 70), (160, 130)])
def test_attention_windows_with_large_heads(d, window, decode_path):
    # the 16-rows-a-wave kernel (head sizes above 128) and the 32-row one, portions longer than a tile of rows, a
    # window that is no multiple of the key tile, pages in front of the window given back
    run_attention(H=4, Hk=2, d=d, P_=16, lens=[400, 230, 90], rows_per_seg=[1, 150, 70], window=window, seed=d)
    run_attention(H=2, Hk=1, d=d, P_=8, lens=[333, 77], rows_per_seg=[100, 1], window=window, seed=d + 1)


@pytest.mark.parametrize("P_", [16, 32, 64, 128])
@pytest.mark.parametrize("d", [128, 64])
def test_attention_of_whole_tiles_of_128_rows(P_, d):
    """Heads of 128 and of 64 in portions that fill tiles of 128 rows: the kernel that takes such a tile a block (keys and values
    by direct loads into LDS, one page per 16 keys).  Several requests, history in front of a portion, rows and keys
    that are no multiple of a tile, one and several key tiles, every page size it takes."""
    run_attention(H=4, Hk=2, d=d, P_=P_, lens=[640, 300, 128], rows_per_seg=[384, 300, 128], seed=P_)
    run_attention(H=8, Hk=8, d=d, P_=P_, lens=[1000, 257, 1], rows_per_seg=[250, 257, 1], seed=P_ + 1)
    run_attention(H=2, Hk=1, d=d, P_=P_, lens=[2500], rows_per_seg=[2500 - 1277], seed=P_ + 2)


@pytest.mark.parametrize("d", [128, 64])
def test_attention_of_whole_tiles_at_the_head_counts_of_an_8b_model(d):
    # 32 heads over 8 kv heads (heads of a kv head share an XCD in the kernel's order of blocks); portions that end in
    # a short tile, that begin at position 0 and deep inside a sequence, and one of a single tile
    run_attention(H=32, Hk=8, d=d, P_=16, lens=[700, 129, 4100, 128], rows_per_seg=[700, 129, 300, 70], seed=3)
    # tiles of 64 rows on average: still the 128-row kernel; one row less on average: the 64-row kernels take over
    run_attention(H=8, Hk=2, d=d, P_=16, lens=[300, 300, 500], rows_per_seg=[64, 64, 64], seed=4)
    run_attention(H=8, Hk=2, d=d, P_=16, lens=[300, 300, 500], rows_per_seg=[64, 63, 64], seed=5)


@pytest.mark.parametrize("window", [1, 37, 128, 200, 1000])
@pytest.mark.parametrize("d", [128, 64])
def test_attention_of_whole_tiles_with_windows(window, d):
    # windows that end inside the first key tile, that span several, that are wider than the keys; pages in front of
    # the window given back (the spare page, full of NaN, stands in); NaN beyond the last key
    run_attention(H=4, Hk=2, d=d, P_=16, lens=[900, 260], rows_per_seg=[500, 260], window=window, seed=window,
                  stale=float("nan"))
    run_attention(H=2, Hk=2, d=d, P_=32, lens=[700], rows_per_seg=[300], window=window, seed=window + 1,
                  stale=float("nan"))


@pytest.mark.parametrize("where", [3, 200, 519, 700])
@pytest.mark.parametrize("d", [128, 64])
def test_attention_of_whole_tiles_when_a_late_key_dwarfs_the_first(where, d):
    """The kernel for tiles of 128 rows keeps a row's first reference for its exponents; a key whose scores lie far
    beyond it (here by hundreds of powers of two) sends the block to its plain loop, whose references move."""
    run_attention(H=4, Hk=2, d=d, P_=16, lens=[768], rows_per_seg=[512], seed=where, loud=(0, where, 40.0))


@pytest.mark.parametrize("range_min", [64, 192, 512])
@pytest.mark.parametrize("d", [128, 64])
def test_attention_of_whole_tiles_with_the_keys_cut_into_ranges(monkeypatch, range_min, d):
    """A step of few tiles over many keys: the keys of every tile are cut into ranges, a block each, and a second
    kernel adds the ranges.  With the smallest range set low so that modest sizes are cut: requests whose tiles have
    very different numbers of keys (some fewer key tiles than ranges: empty ranges), NaN beyond the last key, windows
    (rows that see no key of a range), a key that dwarfs the others in the first and in a later range, 8 ranges."""
    nan = float("nan")
    monkeypatch.setattr(tuned(), "KEY_RANGE_MIN", range_min)
    n = lambda keys, blocks: max(1, min(8, 256 // blocks, max(keys // range_min, min(keys // (range_min // 2), 128 // blocks))))
    run_attention(H=4, Hk=2, d=d, P_=16, lens=[1500, 200, 128], rows_per_seg=[300, 200, 100], seed=range_min, stale=nan,
                  ranges=n(1500, 6 * 4))
    run_attention(H=2, Hk=1, d=d, P_=32, lens=[2500], rows_per_seg=[130], seed=range_min + 1, ranges=n(2500, 2 * 2))
    run_attention(H=4, Hk=2, d=d, P_=16, lens=[1900, 700], rows_per_seg=[250, 128], window=700, seed=range_min + 2,
                  stale=nan, ranges=n(828, 3 * 4))
    run_attention(H=4, Hk=2, d=d, P_=16, lens=[1900], rows_per_seg=[128], window=150, seed=range_min + 3, stale=nan,
                  ranges=n(278, 4))
    for where in (3, 1100, 1499):
        run_attention(H=4, Hk=2, d=d, P_=16, lens=[1500], rows_per_seg=[256], seed=range_min + where,
                      loud=(0, where, 40.0), ranges=n(1500, 2 * 4))


@pytest.mark.parametrize("d", [128, 64])
def test_attention_of_whole_tiles_with_the_keys_cut_into_ranges_at_the_size_from_which_it_is_done(d):
    # 1,024 keys a range while the cut leaves the chip at most half full: 4,500 keys in 4 ranges, 17,000 in 8, 1,000 whole;
    # 2,048 keys a range where it fills the chip: 32 heads x 4 tiles over 4,200 keys in 2 ranges, over 4,000 whole
    run_attention(H=4, Hk=2, d=d, P_=16, lens=[4500], rows_per_seg=[100], seed=1, ranges=4)
    run_attention(H=2, Hk=1, d=d, P_=64, lens=[17000], rows_per_seg=[129], seed=2, ranges=8)
    run_attention(H=4, Hk=2, d=d, P_=16, lens=[1000], rows_per_seg=[100], seed=3, ranges=1)
    run_attention(H=32, Hk=8, d=d, P_=16, lens=[4200], rows_per_seg=[512], seed=4, ranges=2)
    run_attention(H=32, Hk=8, d=d, P_=16, lens=[4000], rows_per_seg=[512], seed=5, ranges=1)


@pytest.mark.parametrize("d", [128, 64])
def test_attention_of_whole_tiles_gives_the_same_bits_every_time(d):
    """The kernel for tiles of 128 rows counts the waits around its MFMAs and LDS reads by hand.  A read whose
    registers the compiler had already given to another value once showed as rows that differ from run to run when
    two blocks shared a compute unit's LDS (heads of 64 run that way).  More blocks than compute units, many times:
    every output equals the first bit by bit (which the other tests hold against the plain implementation at smaller
    sizes); tests/test_kernel_waits.py looks for the pattern itself in the compiler's output."""
    from allpaca_amd.engine.batch import Entry, pack_step
    from allpaca_amd.kernels import ops as kernel_ops
    t = tuned()
    H, Hk, P_, keys, rows = 32, 8, 16, 6144, 2048
    cache, bt, ks, vs = make_cache([keys], Hk, d, P_, BF, seed=d)
    tables = [[list(bt[0, : keys // P_].cpu().numpy())]]
    spare = min(set(range(cache.shape[0])) - {int(p) for p in tables[0][0]})
    step = pack_step([Entry(0, [0] * rows, [])], [keys - rows], [0], tables, torch.device(DEV), [spare],
                     tile_rows=kernel_ops.attention_tile_rows(BF))
    q = gen(rows, H * d, seed=d + 1, scale=2.5, dtype=BF).to(DEV)
    outs = [torch.zeros(rows, H * d, dtype=BF, device=DEV) for _ in range(24)]
    for o in outs:
        assert t.attention_bf16(q, 0, o, H, Hk, d, cache, P_, step.block_tables[0], step)
    first = outs[0].view(torch.int16)
    differ = [i for i, o in enumerate(outs) if not torch.equal(o.view(torch.int16), first)]
    assert not differ, f"runs {differ} differ from the first"
    want = P.attention(f64(q[-3:]).reshape(3, H, d), f64(ks[0]), f64(vs[0]), H, Hk)
    assert np.abs(f64(outs[0][-3:]).reshape(3, H, d) - want).max() < 2.0 ** -7 * np.abs(f64(vs[0])).max() * 0.25 + 2.0 ** -8 * np.abs(want).max()


@pytest.mark.parametrize("d", [16, 64, 128, 192, 256])
@pytest.mark.parametrize("whole", [False, True])
def test_attention_ignores_what_it_does_not_see(monkeypatch, d, whole, decode_path):
    """NaN in every slot beyond a sequence's last key (what a page's last owner may have left there) and in the
    spare page that stands for pages in front of a window: those positions get a weight of 0, and 0 x NaN must
    not reach the output."""
    monkeypatch.setattr(tuned(), "WHOLE_MIN_PAIRS", 1 if whole else 1 << 30)
    nan = float("nan")
    run_attention(H=4, Hk=2, d=d, P_=16, lens=[150, 70, 33, 1, 2049], rows_per_seg=[150, 1, 5, 1, 1], seed=d, stale=nan)
    run_attention(H=4, Hk=2, d=d, P_=8, lens=[300, 203, 90, 61], rows_per_seg=[1, 130, 17, 1], window=45, seed=d, stale=nan)
    run_attention(H=4, Hk=1, d=d, P_=24, lens=[300, 203, 9], rows_per_seg=[1, 66, 9], window=100, seed=d, stale=nan)


def test_attention_long_context_decode_and_portion_over_history(decode_path):
    # the reference's long rows (crates/allpaca-hip/src/lib.rs:23162-23175: 3000 and 1300 keys) and a portion
    # of 70 rows over 2,000 keys of history
    run_attention(H=4, Hk=2, d=128, P_=16, lens=[3000, 1300, 2070], rows_per_seg=[1, 2, 70], seed=1)
    run_attention(H=8, Hk=8, d=128, P_=16, lens=[5000] + [40] * 7, rows_per_seg=[1] * 8, seed=2)


@pytest.mark.parametrize("H,Hk,d,P_,lens,rows,window", [
    (32, 8, 128, 16, [2048, 1, 17, 700, 2047], [1, 1, 1, 1, 1], 0),
    (4, 2, 64, 16, [3000, 5000, 40, 2049], [1, 1, 1, 1], 0),          # several ranges of keys a wave
    (6, 2, 48, 8, [300, 129, 64, 1], [1, 1, 1, 1], 0),
    (20, 1, 32, 24, [100, 260, 64], [1, 1, 1], 0),                     # a group wider than one 16-row tile
    (34, 2, 80, 16, [100, 260], [1, 1], 0),
    (16, 1, 256, 32, [500, 90], [1, 1], 0),                            # the meeting place does not fit: parts and merge
    (4, 2, 32, 16, [300, 200, 90, 2500], [1, 1, 1, 1], 100),
    (4, 4, 16, 16, [300, 200, 90, 1200], [1, 1, 1, 1], 1000),
    (4, 2, 64, 8, [4000, 70, 1500, 1], [1, 1, 1, 1], 0),               # a wave's range in several pieces (pages of 8)
    (4, 2, 32, 8, [4000, 300], [1, 1], 3000),
    (8, 2, 128, 16, [900, 133, 400], [1, 40, 1], 5),                    # decode rows beside a portion
])
def test_attention_decode_by_one_block_a_row_and_kv_head(monkeypatch, H, Hk, d, P_, lens, rows, window):
    """The decode kernel in which the waves of one block take all keys of a (row, kv head) and finish its heads
    themselves (chosen from 256 such pairs on; forced here) against the plain attention."""
    monkeypatch.setattr(tuned(), "WHOLE_MIN_PAIRS", 1)
    run_attention(H=H, Hk=Hk, d=d, P_=P_, lens=lens, rows_per_seg=rows, window=window, seed=H + d)


def test_attention_decode_of_many_rows_takes_the_one_block_kernel_by_itself():
    # 40 rows x 8 kv heads: above the threshold without forcing; contexts from 1 to 2,100 keys
    lens = [1 + (i * 211) % 2100 for i in range(40)]
    run_attention(H=16, Hk=8, d=64, P_=16, lens=lens, rows_per_seg=[1] * 40, seed=3)


def test_attention_finds_a_far_key_in_every_path(monkeypatch):
    t = tuned()
    from allpaca_amd.engine.batch import Entry, pack_step
    H, Hk, d, P_, n = 4, 2, 64, 16, 900
    for rows, whole in ((1, False), (40, False), (1, True)):
        monkeypatch.setattr(t, "WHOLE_MIN_PAIRS", 1 if whole else 1 << 30)
        cache, bt, ks, vs = make_cache([n], Hk, d, P_, BF, seed=9)
        key = 17
        page, slot = int(bt[0, key // P_]), key % P_
        cache[page, 0, :, slot] = 0.0
        cache[page, 0, :, slot, 5] = 30.0
        q = torch.zeros(rows, H * d, dtype=BF, device=DEV)
        for h in range(H):
            q[-1, h * d + 5] = 30.0
        step = pack_step([Entry(0, [0] * rows, [])], [n - rows], [0],
                         [[list(bt[0, : -(-n // P_)].cpu().numpy())]], torch.device(DEV), [0])
        out = torch.zeros(rows, H * d, dtype=BF, device=DEV)
        assert t.attention_bf16(q, 0, out, H, Hk, d, cache, P_, step.block_tables[0], step)
        for h in range(H):
            want = vs[0][key, h // 2].float()
            assert torch.allclose(out[-1, h * d:(h + 1) * d].float().cpu(), want, atol=2.0 ** -7 * 4)


@pytest.mark.parametrize("parts", [4, 5, 6, 13, 32])
@pytest.mark.parametrize("window", [0, 700])
def test_attention_decode_with_rows_of_very_different_lengths(monkeypatch, parts, window, decode_path):
    """Every row's own keys go into the launch's number of ranges: rows of 1 to 6,000 keys in one launch, with counts
    of ranges that do not fill the last block, ranges far longer than a wave keeps page ids for (pages of 8), and a
    window whose first key lies inside a range."""
    if decode_path == "last block merges" or decode_path == "merge kernel":
        monkeypatch.setattr(tuned(), "_decode_parts", lambda pairs, span: parts)
    run_attention(H=8, Hk=2, d=64, P_=8, lens=[6000, 1, 63, 64, 65, 1500, 2063, 129], rows_per_seg=[1] * 8,
                  window=window, seed=parts)


def test_attention_decode_many_launches_leave_the_counters_at_zero():
    """The counters that tell the last block of a (row, kv head) are set back by that block: launch after launch on
    the same counters, with other batch sizes, contexts and head counts in between, gives the right rows."""
    t = tuned()
    for rep in range(3):
        run_attention(H=8, Hk=2, d=128, P_=16, lens=[2049, 700, 33, 1], rows_per_seg=[1, 1, 1, 1], seed=rep)
        run_attention(H=4, Hk=4, d=64, P_=8, lens=[5000], rows_per_seg=[1], seed=10 + rep)
        run_attention(H=32, Hk=8, d=128, P_=16, lens=[2048 + 7 * i for i in range(8)], rows_per_seg=[1] * 8, seed=20 + rep)
    for dev_counters in t._counters.values():
        for c in dev_counters:
            assert int(c.abs().max()) == 0
