"""Pages beyond 4 GiB: a cache of 70,000 pages at the page size of an 8B model (8 kv heads of 128, 16 positions:
64 KiB a page and layer, 4.4 GiB in all), block tables that point past page 65,536, where a byte offset no longer
fits 32 bits.  The kernels that write pages (rotation and cache write alone and inside the product for q, k, v) and
those that read them (decode attention in its three ways of merging, both kernels for prompt portions) against the
float64 reference and against the same kernels on a small cache."""
import numpy as np
import pytest
import torch

import plain_llama as P
from test_kernels_plain import DEV, f64, gen
from test_kernels_tuned import BF, pack, run_attention, tuned

pytestmark = pytest.mark.gpu

PAGES, HK, D, PT = 70000, 8, 128, 16
FIRST_HIGH = 65600          # every page used lies at or beyond this id: more than 4 GiB into the tensor


@pytest.fixture(scope="module")
def big():
    free, _ = torch.cuda.mem_get_info()
    need = PAGES * 2 * HK * PT * D * 2
    if free < need + (4 << 30):
        pytest.skip(f"{need / 2**30:.1f} GiB of device memory for the large cache are not free")
    cache = torch.zeros((PAGES, 2, HK, PT, D), dtype=BF, device=DEV)
    assert cache[FIRST_HIGH].data_ptr() - cache.data_ptr() > 1 << 32
    yield cache
    del cache
    torch.cuda.empty_cache()


def high_page(p):
    """Where page p of a small cache goes in the large one (scattered, all beyond FIRST_HIGH)."""
    return PAGES - 1 - 3 * p


def relocate_into(big):
    def relocate(cache, bt):
        n = cache.shape[0]
        assert high_page(n - 1) >= FIRST_HIGH
        where = torch.tensor([high_page(p) for p in range(n)], device=DEV)
        big[where] = cache
        return big, torch.from_numpy(np.vectorize(high_page)(bt.cpu().numpy()).astype(np.int32)).to(DEV)
    return relocate


def test_prompt_portions_read_pages_beyond_4_gib(big):
    # tiles of 128 rows, a block a tile and head; with the keys of a tile cut into ranges; short tiles on the 64-row kernel
    run_attention(32, HK, D, PT, lens=[700, 300], rows_per_seg=[700, 129], seed=1, relocate=relocate_into(big))
    run_attention(32, HK, D, PT, lens=[9000], rows_per_seg=[256], seed=2, ranges=4, relocate=relocate_into(big))
    run_attention(32, HK, D, PT, lens=[500, 300, 200], rows_per_seg=[33, 20, 7], seed=3, relocate=relocate_into(big))


@pytest.mark.parametrize("way", ["last block merges", "merge kernel", "whole"])
def test_decode_rows_read_pages_beyond_4_gib(big, way, monkeypatch):
    t = tuned()
    monkeypatch.setattr(t, "LAST_BLOCK_MERGES", way == "last block merges")
    monkeypatch.setattr(t, "WHOLE_MIN_PAIRS", 1 if way == "whole" else 1 << 30)
    run_attention(32, HK, D, PT, lens=[3000, 150, 2049, 17], rows_per_seg=[1, 1, 1, 1], seed=4, relocate=relocate_into(big))


@pytest.mark.parametrize("M,fused", [(8, False), (70, False), (8, True), (64, True)])
def test_keys_and_values_are_written_into_pages_beyond_4_gib(big, M, fused):
    """Rotation and cache write (alone: M rows of a finished product; fused: inside the product for q, k, v, the streaming
    kernel at 8 rows and the finishing kernel of the tiled product at 64): the pages written far into the large cache
    hold, bit for bit, what the same call writes into a small one, and nothing else was touched."""
    from allpaca_amd.kernels import ops
    H, K = 32, 512
    N = (H + 2 * HK) * D
    rng = np.random.default_rng(M)
    max_blocks = 12
    pos_list = sorted(rng.choice(max_blocks * PT, size=M, replace=False).tolist())
    seg_list = [i % 3 for i in range(M)]
    pos = torch.tensor(pos_list, dtype=torch.int32, device=DEV)
    seg = torch.tensor(seg_list, dtype=torch.int32, device=DEV)
    small_bt = rng.permutation(3 * max_blocks).reshape(3, max_blocks).astype(np.int32)
    ang = np.arange(max_blocks * PT)[:, None] * (1.0 / 300.0 ** (np.arange(D // 2) / (D // 2)))[None, :]
    table = torch.from_numpy(np.stack([np.cos(ang), np.sin(ang)], 1).astype(np.float32)).to(DEV)
    w = pack(gen(N, K, seed=3, dtype=BF).to(DEV))
    a = gen(M, K, seed=1, dtype=BF, scale=2.0).to(DEV)
    qkv0 = gen(M, N, seed=2, dtype=BF).to(DEV)
    big.zero_()
    out = []
    for cache, bt in ((torch.zeros(3 * max_blocks, 2, HK, PT, D, dtype=BF, device=DEV), small_bt),
                      (big, np.vectorize(high_page)(small_bt).astype(np.int32))):
        bt = torch.from_numpy(bt).to(DEV)
        qkv = qkv0.clone()
        if fused:
            assert ops.qkv_rope_write(a, None, w, qkv, H, HK, D, table, pos, seg, bt, cache, PT)
        else:
            ops.rope_kv_write(qkv, 0, H * D, (H + HK) * D, H, HK, D, D, table, pos, seg, bt, cache, PT)
        out.append((qkv, cache))
    (q_small, c_small), (q_big, c_big) = out
    assert torch.equal(q_small[:, :H * D], q_big[:, :H * D])
    where = torch.tensor([high_page(p) for p in range(3 * max_blocks)], device=DEV)
    assert torch.equal(c_big[where], c_small) and int((c_small != 0).sum()) > 0
    c_big[where] = 0
    assert int(c_big[FIRST_HIGH - 64:].ne(0).sum()) == 0 and int(c_big[:4096].ne(0).sum()) == 0
