"""Kernel paths that only the sizes of real models select (a vocabulary of 128,256: the argmax in pieces, the
streaming product with two bands a block, the sampler over a long row), each against the plain implementation or a
float64 product.  The tiny configurations never reach them."""
import os

import numpy as np
import pytest
import torch

import helpers as H

import plain_llama as P
from test_kernels_plain import DEV, f64, gen
from test_kernels_tuned import BF, check, pack, tuned

pytestmark = pytest.mark.gpu

VOCAB = 128256


def ops():
    from allpaca_amd.kernels import ops as o
    return o


@pytest.mark.parametrize("V", [8192, 8193, VOCAB])
def test_argmax_in_pieces_takes_the_first_maximum(V):
    """From 8,192 columns on a row is cut into 64 pieces and a second kernel takes the first maximum of the pieces'
    (crates/allpaca-core/src/sampling.rs:215-234: strict >, the lowest index among equals, token 0 when nothing is
    above -inf)."""
    o = ops()
    piece = -(-V // 64)
    R = 12
    lg = gen(R, V, seed=V).clone()
    top = float(lg.max()) + 1.0
    lg[0, 5 * piece + 3] = top
    lg[0, 40 * piece + 1] = top                  # equal maxima in two pieces: the earlier piece wins
    lg[1, 40 * piece + 1] = top
    lg[1, 40 * piece + 300] = top                # ... and inside one piece, in different threads
    lg[2, :] = float("-inf")                     # nothing above -inf: token 0
    lg[3, V - 1] = top                           # the last column (the last piece is the short one)
    lg[4, 0] = top
    lg[5, :] = float("nan")                      # no comparison with NaN holds: token 0
    lg[6, 17 * piece: 18 * piece] = float("nan")
    lg[6, 63 * piece] = top                      # first column of the last piece, behind a piece of NaN
    lg[7, 9 * piece - 1] = top
    lg[7, 9 * piece] = top                       # neighbours across a border between pieces
    lg[8, 123] = float("inf")
    lg[8, 60 * piece] = float("inf")
    lg[9, :] = -3.0                              # all equal: index 0
    out = torch.full((R,), -1, dtype=torch.int32, device=DEV)
    o.argmax_rows(lg.to(DEV), out)
    want = [P.argmax(row) for row in lg.numpy()]
    assert out.cpu().tolist() == want
    assert want[:10] == [5 * piece + 3, 40 * piece + 1, 0, V - 1, 0, 0, 63 * piece, 9 * piece - 1, 123, 0]


def _columns(N, rng, n=3000):
    """A sample of output columns that holds the first and last bands and both sides of a block's border."""
    fixed = list(range(0, 48)) + list(range(N - 40, N)) + list(range(N // 2 - 20, N // 2 + 20))
    return np.unique(np.concatenate([np.asarray(fixed), rng.integers(0, N, size=n)]))


@pytest.mark.parametrize("K", [4096, 3072])
def test_products_with_a_vocabulary_of_output_columns(K):
    """The head of an 8B (K = 4096) and a 3B (K = 3072) model: [128256, K].  Up to 16 rows the streaming kernel
    takes two bands a block (from 32,768 columns on); more rows go to the tiled kernel, whole or with K in slices.
    Every path against the float64 product on a sample of columns."""
    t = tuned()
    N = VOCAB
    g = torch.Generator(device=DEV).manual_seed(K)
    w = (torch.randn((N, K), generator=g, device=DEV) * 0.05).to(BF)
    wp = pack(w)
    rng = np.random.default_rng(K)
    cols = _columns(N, rng)
    w64 = f64(w[torch.from_numpy(cols).to(DEV)])
    for M in (1, 8, 16, 17, 64, 300):
        a = gen(M, K, seed=M, dtype=BF).to(DEV)
        want = f64(a) @ w64.T
        for out_dtype in ((BF, torch.float32) if M in (8, 64) else (torch.float32,)):
            out = torch.full((M, N), 7.0, dtype=out_dtype, device=DEV)
            t.gemm_bf16(a, wp, out)
            check(f64(out[:, torch.from_numpy(cols).to(DEV)]), want, out_dtype)
            # nothing is left unwritten anywhere in the row
            assert not bool((out == 7.0).all(dim=0).any())
    # rows together equal each row alone, bit for bit, on the two-band kernel too
    a = gen(16, K, seed=99, dtype=BF).to(DEV)
    tog = torch.empty(16, N, dtype=torch.float32, device=DEV)
    t.gemm_bf16(a, wp, tog)
    alone = torch.empty(1, N, dtype=torch.float32, device=DEV)
    t.gemm_bf16(a[5:6], wp, alone)
    assert torch.equal(alone[0], tog[5])


@pytest.mark.parametrize("one_block", [False, True], ids=["many blocks a row", "one block a row"])
def test_sampler_over_a_real_vocabulary(one_block):
    """temperature / top-k / top-p over 128,256 logits against the plain sampler (crates/allpaca-core/src/
    sampling.rs:24-67, 215-331)."""
    o = ops()
    V, R = VOCAB, 14
    rng = np.random.default_rng(5)
    lg = gen(R, V, seed=77) * 3.0
    lg[0, 3] = lg[0, 90000] = lg[0, V - 1] = 20.0          # ties at the top, far apart
    lg[1, :] = float("nan")                                 # degenerate: token 0
    lg[2, 100000:] = float("-inf")
    temps = np.asarray([0.7, 1.0, 0.9, 0.0, 1.5, 0.8, 0.8, 0.8, 1.0, 0.3, 1.0, 2.0, 0.8, 1.0], np.float32)
    ks = np.asarray([0, 5, 0, 0, 40, 40, 1, 2000, 0, 0, 100000, 0, 40, 0], np.int32)
    ps = np.asarray([1.0, 1.0, 0.9, 1.0, 0.95, 0.5, 1.0, 0.95, 0.1, 1.0, 0.99, 0.0, 0.95, 0.999], np.float32)
    us = rng.random(R).astype(np.float32)
    us[5] = 0.0
    us[8] = 0.99999994
    out = torch.empty(R, dtype=torch.int32, device=DEV)
    o.sample_rows(lg.to(DEV), torch.from_numpy(temps).to(DEV), torch.from_numpy(ks).to(DEV),
                  torch.from_numpy(ps).to(DEV), torch.from_numpy(us).to(DEV), out, one_block=one_block)
    got = out.cpu().tolist()
    lgn = lg.numpy()
    bad = []
    for r in range(R):
        want = P.sample(lgn[r], float(temps[r]), int(ks[r]), float(ps[r]), float(us[r]))
        if got[r] != want:
            # a draw within rounding of the border between two candidates may fall either way (the sum over
            # 128,256 probabilities in float32 against float64): the neighbour that a nudged draw gives is accepted
            near = {P.sample(lgn[r], float(temps[r]), int(ks[r]), float(ps[r]), float(us[r]) + e) for e in (-2e-5, 2e-5)}
            if got[r] not in near:
                bad.append((r, got[r], want))
    assert not bad, bad


def test_sampler_over_more_than_a_million_logits():
    """Beyond 2^20 logits the sort key (32 bits of value, 21 of id) takes a fifth digit of 13 bits: the sampler with many
    blocks a row against the one with one block a row (and against the plain sampler on the rows that are cheap there:
    top-k leaves few candidates)."""
    o = ops()
    V, R = (1 << 20) + 4099, 6
    lg = gen(R, V, seed=5) * 3.0
    lg[0, 7] = lg[0, V - 1] = lg[0, V // 2] = 25.0           # ties at the top, as far apart as ids get
    lg[1] = torch.round(lg[1] * 4) / 4                        # runs of equal values everywhere
    temps = np.asarray([0.7, 1.0, 0.9, 1.2, 0.8, 1.0], np.float32)
    ks = np.asarray([0, 0, 40, 5, 0, 3000], np.int32)
    ps = np.asarray([1.0, 0.9, 0.95, 1.0, 0.5, 0.99], np.float32)
    us = np.random.default_rng(9).random(R).astype(np.float32)
    d = [torch.from_numpy(a).to(DEV) for a in (temps, ks, ps, us)]
    lgd = lg.to(DEV)
    many = torch.empty(R, dtype=torch.int32, device=DEV)
    one = torch.empty(R, dtype=torch.int32, device=DEV)
    o.sample_rows(lgd, *d, many)
    o.sample_rows(lgd, *d, one, one_block=True)
    assert many.cpu().tolist() == one.cpu().tolist()
    lgn = lg.numpy()
    for r in (2, 3):
        assert int(many[r]) == P.sample(lgn[r], float(temps[r]), int(ks[r]), float(ps[r]), float(us[r]))


def test_a_folder_at_the_widths_of_a_3b_model_through_the_front_door(tmp_path):
    """config.json + model.safetensors of two layers at the widths of Llama-3.2-3B (hidden 3072, 24 heads over 8 of
    128, feed-forward 8192, vocabulary 128,256, tied head: 1.2 GB in bfloat16) written tensor by tensor, loaded by
    `Engine(folder)` with a pool sized from free device memory, and run: greedy tokens are the plain implementation's
    choice or within bfloat16's noise of it."""
    import resource
    import time
    from allpaca_amd.config import preset
    from allpaca_amd.engine import Engine
    from allpaca_amd.sampling import GenerationParams
    from allpaca_amd.weights import write_model_folder
    cfg_json = dict(preset("llama-3.2-3b"), num_hidden_layers=2)
    folder = str(tmp_path / "m3b")
    assert write_model_folder(folder, cfg_json, 11, torch.bfloat16, keep_tensors=False, device=DEV) is None
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    torch.cuda.reset_peak_memory_stats()
    free_before, _ = torch.cuda.mem_get_info()
    t0 = time.time()
    eng = Engine(folder, dtype="bfloat16", max_active_requests=4, kv_reserve_bytes=8 << 30)
    load_s = time.time() - t0
    weights = sum(os.path.getsize(os.path.join(folder, f)) for f in os.listdir(folder))
    pool = eng.runner.cache.paged_groups[0].pool.num_pages
    # the pool: what 4 requests of the longest context need (131,072 positions each), since that fits this card; with
    # a budget given in bytes, floor(budget / bytes of a page over both layers) less the spare page
    assert pool == 4 * (131072 // 16)
    page = 2 * 2 * 8 * 16 * 128 * 2
    assert Engine.pages_that_fit(eng.model, type(eng.config)(kv_bytes=1000 * page + 5, max_active_requests=4)) == 999
    prompts = [H.random_tokens(VOCAB, n, seed=n) for n in (5, 40)]
    outs = eng.generate(prompts, GenerationParams(max_tokens=4, temperature=0.0))
    cfg, w = P.read_model_folder(folder)
    for p, o in zip(prompts, outs):
        lg = P.llama_forward(cfg, w, p + o.token_ids[:-1])[len(p) - 1:]
        for j, t in enumerate(o.token_ids):
            assert lg[j].max() - lg[j][t] <= 0.02 * np.abs(lg[j]).max(), (j, t)
    peak_dev = torch.cuda.max_memory_allocated()
    peak_host = resource.getrusage(resource.RUSAGE_SELF).ru_maxrss * 1024
    print(f"\n3B widths, 2 layers: file {weights / 2**30:.2f} GiB, load {load_s:.2f} s, device peak "
          f"{peak_dev / 2**30:.2f} GiB (pool {eng.runner.storage.bytes() / 2**30:.2f} GiB), host peak rss "
          f"{peak_host / 2**30:.2f} GiB, free before {free_before / 2**30:.1f} GiB")
    # the weights once, the pool, and working memory: never the model twice over
    assert peak_dev <= eng.runner.storage.bytes() + weights + (3 << 30)
