"""Host-side rules that choose a kernel's shape from a step's sizes (no GPU): into how many ranges the keys of a tile
of prompt rows are cut, and which launches the sampler is told to leave out."""
from types import SimpleNamespace

import pytest


def _step(segments, tile=128):
    """A step of prompt portions: (position of the first row, rows) per segment."""
    n_tiles = sum(-(-n // tile) for _, n in segments if n > 1)
    return SimpleNamespace(n_tiles=n_tiles, host_pos0=[p for p, _ in segments], host_rows=[n for _, n in segments])


def test_key_ranges_of_a_step():
    from allpaca_amd.kernels import tuned
    ks = tuned._key_splits
    # a chunk of 512 rows at 32 heads is 128 blocks: cut in two from 4,096 keys on, never more (256 compute units)
    assert ks(_step([(0, 512)]), 32, 0) == 1
    assert ks(_step([(2048 - 512, 512)]), 32, 0) == 1
    assert ks(_step([(4096 - 512, 512)]), 32, 0) == 2
    assert ks(_step([(131072 - 512, 512)]), 32, 0) == 2
    # 128 rows are 32 blocks: ranges of 1,024 keys while the chip stays half empty, of 2,048 beyond, 8 at most
    assert [ks(_step([(n - 128, 128)]), 32, 0) for n in (1000, 2048, 3072, 4096, 8192, 16384, 65536)] == [1, 2, 3, 4, 4, 8, 8]
    # a whole-prompt step has blocks enough
    assert ks(_step([(0, 2048)]), 32, 0) == 1 and ks(_step([(30720, 2048)]), 32, 0) == 1
    # 64 heads: a chunk of 512 fills the chip by itself; 8 heads: 32 blocks
    assert ks(_step([(32768 - 512, 512)]), 64, 0) == 1
    assert ks(_step([(8192 - 512, 512)]), 8, 0) == 4
    # the longest prompt of the step counts, single rows (decoding requests) do not; a window bounds the keys
    assert ks(_step([(100, 128), (8000, 128), (50000, 1)]), 32, 0) == 3
    assert ks(_step([(50000, 1), (10, 128)]), 32, 0) == 1
    assert ks(_step([(32768 - 128, 128)]), 32, 1000) == 1
    assert ks(_step([(32768 - 128, 128)]), 32, 4096) == 4
    # nothing known of the step's positions: no cutting
    assert ks(SimpleNamespace(n_tiles=1), 32, 0) == 1


def test_key_ranges_can_be_switched_off(monkeypatch):
    from allpaca_amd.kernels import tuned
    monkeypatch.setattr(tuned, "KEY_SPLITS_MAX", 0)
    assert tuned._key_splits(_step([(32768 - 128, 128)]), 32, 0) == 1


@pytest.mark.parametrize("rules,want", [
    # (temperature, top-k, top-p) per row -> (some top-k, some top-p, few survivors everywhere)
    ([(0.8, 40, 0.95)], (True, True, True)),
    ([(0.8, 0, 1.0)], (False, False, False)),
    ([(0.8, 0, 0.9), (0.0, 0, 1.0)], (False, True, False)),
    ([(0.8, 40, 1.0), (0.0, 0, 1.0)], (True, False, True)),      # a greedy row needs no launch of its own
    ([(0.8, 2000, 1.0)], (True, False, False)),
    ([(0.8, 40, 0.95), (0.7, 0, 0.95)], (True, True, False)),
])
def test_what_the_sampler_tells_the_kernels(monkeypatch, rules, want):
    """`Sampler.launch` passes on which cuts its rows ask for, so that the kernels leave out the launches nobody needs."""
    import torch
    from allpaca_amd.kernels import ops
    from allpaca_amd.sampling import GenerationParams
    from allpaca_amd.sampling import sampler as S
    seen = {}

    def fake_sample_rows(logits, t, k, p, u, out, **kw):
        seen.update(kw)

    monkeypatch.setattr(ops, "sample_rows", fake_sample_rows)
    monkeypatch.setattr(S.Sampler, "_upload", lambda self, params, indices: torch.zeros(4, 64))
    monkeypatch.setattr(torch.Tensor, "pin_memory", lambda self: self)
    monkeypatch.setattr(torch.cuda, "Event", lambda *a, **k: SimpleNamespace(record=lambda: None, synchronize=lambda: None))
    s = S.Sampler(torch.device("cpu"), 0)
    params = [GenerationParams(max_tokens=1, temperature=t, top_k=k, top_p=p) for t, k, p in rules]
    s.launch(torch.zeros(len(rules), 16), params, [0] * len(rules))
    assert (seen["any_top_k"], seen["any_top_p"], seen["few_after_top_k"]) == want


def test_ranges_the_decode_attention_cuts_a_rows_keys_into():
    """Four ranges a block, as many blocks a (row, kv head) pair as keep the launch within the chip's compute units,
    and no range under 64 keys."""
    from allpaca_amd.kernels import tuned as t
    got = {(n, ctx): t._decode_parts(n * 8, ctx) for n, ctx in
           [(1, 2048), (4, 2048), (8, 2048), (8, 2063), (12, 2048), (16, 2048), (24, 2048), (8, 8192), (16, 8192),
            (1, 32768), (8, 512), (1, 10), (40, 2048)]}
    assert got == {(1, 2048): 32, (4, 2048): 32, (8, 2048): 16, (8, 2063): 16, (12, 2048): 8, (16, 2048): 8,
                   (24, 2048): 4, (8, 8192): 16, (16, 8192): 8, (1, 32768): 128, (8, 512): 8, (1, 10): 1, (40, 2048): 4}
    for pairs in (1, 8, 64, 100, 255, 256, 1000):
        for span in (1, 64, 65, 2048, 1 << 20):
            parts = t._decode_parts(pairs, span)
            blocks = pairs * -(-parts // t.WHOLE_WAVES)
            assert parts >= 1 and (blocks <= max(pairs, t.CHIP_UNITS)) and (parts == 1 or span / parts >= 32)


def test_the_executors_rules_are_the_wrappers_rules():
    """The compiled plan executor (csrc/host/rules.h) chooses slices of K, keys a wave and ranges of keys by the same
    rules as the Python wrappers of the kernels: held against each other over the shapes either may meet."""
    from allpaca_amd.kernels import host, tuned
    L = host.load()
    for M in (17, 24, 32, 48, 64, 100, 128, 129, 200, 256, 384, 500, 512, 640, 768, 1000, 1024, 1025, 2048):
        for N in (192, 1000, 2048, 3072, 4096, 5120, 6144, 8192, 14336, 16384, 28672, 57344, 128256):
            for K in (120, 192, 512, 2048, 3072, 4096, 8192, 14336, 28672):
                assert L.apc_host_rule_tiled_k_split(M, N, K) == tuned._tiled_k_split(M, N, K), (M, N, K)
    for pairs in (1, 2, 3, 8, 12, 16, 24, 31, 64, 100, 255, 256, 257, 2040):
        for span in (1, 63, 64, 65, 2048, 2049, 8192, 32768, 131072):
            assert L.apc_host_rule_decode_parts(pairs, span) == tuned._decode_parts(pairs, span), (pairs, span)
    for rows in (2, 100, 128, 129, 256, 512, 1024, 2048):
        for pos0 in (0, 500, 1920, 3584, 8000, 32640, 130000):
            for heads in (4, 8, 24, 32, 64):
                for window in (0, 1000, 4096):
                    step = _step([(pos0, rows), (7, 1)])
                    want = tuned._key_splits(step, heads, window)
                    got = L.apc_host_rule_key_splits(step.n_tiles, heads, pos0 + rows, window, tuned.KEY_SPLITS_MAX,
                                                     tuned.KEY_RANGE_MIN)
                    assert got == want, (rows, pos0, heads, window)
