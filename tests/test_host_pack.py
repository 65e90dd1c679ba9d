"""The C++ step packer (csrc/host/pack.cpp) against the Python one (engine/batch.py::pack_step), which the kernel
tests and models with positions on several axes use: the same buffer, array by array, for random steps over a
cache with a windowed group; and what it refuses (no GPU)."""
import ctypes

import numpy as np
import pytest
import torch

from allpaca_amd.cache import CacheManager, OutOfPages
from allpaca_amd.engine.batch import ARRAYS, Entry, StepLayout, pack_step
from allpaca_amd.kernels import host as H
from allpaca_amd.parts import PagedKV


def flat(cm, entries):
    ids = np.asarray([cm.id_of(e.seq) for e in entries], dtype=np.int64)
    n_tok = np.asarray([len(e.tokens) for e in entries], dtype=np.int32)
    toks = np.asarray(sum([list(e.tokens) for e in entries], []), dtype=np.int32)
    n_want = np.asarray([len(e.want) for e in entries], dtype=np.int32)
    wants = np.asarray(sum([list(e.want) for e in entries], []), dtype=np.int32)
    return ids, n_tok, toks, n_want, wants


def prepare(cm, entries, vocab=1000, max_positions=10000):
    ids, n_tok, toks, n_want, wants = flat(cm, entries)
    f = H.ApcStepFinding()
    code = H.load().apc_step_prepare(cm.handle, vocab, max_positions, len(entries), ids.ctypes.data, n_tok.ctypes.data,
                                     toks.ctypes.data, n_want.ctypes.data, wants.ctypes.data, ctypes.byref(f))
    return code, (f.what, f.entry, f.value, f.extra)


@pytest.mark.parametrize("seed", range(6))
def test_the_same_buffer_as_the_python_packer(seed):
    rng = np.random.default_rng(seed)
    L = H.load()
    tile = int(rng.choice([4, 8, 128]))
    cm = CacheManager([PagedKV(2, 32), PagedKV(2, 32, window=9), PagedKV(2, 32)], 4, [120, 60], 6)
    live = {}
    for step in range(40):
        for name in "abcdef":
            if name not in live and rng.random() < 0.3:
                cm.admit(name)
                live[name] = 0
        entries = []
        for name in list(live):
            if rng.random() < 0.25:
                continue
            n = 1 if rng.random() < 0.5 else int(rng.integers(2, 30))
            want = sorted(set(rng.integers(0, n, size=int(rng.integers(0, 3))).tolist()))
            entries.append(Entry(name, rng.integers(0, 1000, size=n).tolist(), want))
        if not entries:
            continue
        code, finding = prepare(cm, entries)
        if code == 7:       # out of pages: nothing was taken; someone ends
            victim = max(live, key=live.get)
            cm.release(victim)
            del live[victim]
            continue
        assert code == 0, finding
        pos0 = [cm.length(e.seq) for e in entries]
        slots = [cm.slot_of(e.seq) for e in entries]
        tables = [[cm.block_table(e.seq, g) for e in entries] for g in range(2)]
        want = pack_step(entries, pos0, slots, tables, torch.device("cpu"), [120, 60], tile_rows=tile)
        ids, n_tok, toks, n_want, wants = flat(cm, entries)
        p, out, pad = H.ApcPacked(), np.full(1 << 14, -7, np.int32), np.asarray([120, 60], np.int32)
        assert L.apc_pack_step(cm.handle, len(entries), ids.ctypes.data, n_tok.ctypes.data, toks.ctypes.data,
                               n_want.ctypes.data, wants.ctypes.data, tile, 1, pad.ctypes.data, out.ctypes.data, out.size,
                               ctypes.byref(p)) == 0
        lay = StepLayout(p.T, p.S, p.R, p.n_decode, p.n_tiles, 1, list(p.table_width[:2]))
        assert lay.total == p.total and [lay.span[a][0] for a in ARRAYS[:11]] == list(p.off)
        got = lay.info(torch.from_numpy(out[:p.total].copy()), [], [], [], [], 0, p.n_decode == p.T)
        for name in ARRAYS[:11]:
            a, b = getattr(want, name), getattr(got, name)
            if a is None or b is None:
                assert (a is None or a.numel() == 0) and (b is None or b.numel() == 0), name
            else:
                assert torch.equal(a, b), name
        for g in range(2):
            assert torch.equal(want.block_tables[g], got.block_tables[g])
        assert (p.max_decode_context, p.max_context, p.max_rows) == (want.max_decode_context, want.max_context, want.max_rows)
        assert L.apc_step_commit(cm.handle, len(entries), ids.ctypes.data, n_tok.ctypes.data) == 0
        cm.check()
        for e in entries:
            live[e.seq] += len(e.tokens)
            if live[e.seq] > 90:
                cm.release(e.seq)
                del live[e.seq]
    for name in list(live):
        cm.release(name)
    cm.check()
    assert cm.free_pages(0) == 120 and cm.free_pages(1) == 60


def test_what_the_packer_refuses():
    cm = CacheManager([PagedKV(2, 32)], 4, 5, 3)
    cm.admit("a")
    cm.admit("b")
    ok = [Entry("a", [1, 2, 3], [2]), Entry("b", [4], [0])]
    assert prepare(cm, [Entry("a", [], [])])[1][:2] == (3, 0)                       # no tokens
    assert prepare(cm, [ok[0], Entry("b", [4, 1000], [0])])[1][:3] == (4, 1, 1000)   # a token outside the vocabulary
    assert prepare(cm, [Entry("a", [1, 2], [2])])[1][:3] == (5, 0, 2)                # a wanted place outside the tokens
    assert prepare(cm, ok, max_positions=2)[1][:3] == (6, 0, 2)                      # a position beyond the limit
    assert cm.free_pages() == 5                                                      # nothing was taken by any of them
    # pages for all or for none: 6 are needed, 5 are there
    assert prepare(cm, [Entry("a", [1] * 12, []), Entry("b", [1] * 9, [])])[1] == (7, 0, 6, 5)
    assert cm.free_pages() == 5 and cm.block_table("a", 0) == []
    assert prepare(cm, ok)[0] == 0 and cm.free_pages() == 3
    with pytest.raises(OutOfPages):
        cm.reserve("b", 30)
