"""The compiled plan executor (csrc/host/exec.cpp) against the same model walked part by part in Python: the same
kernels with the same arguments, so the logits are equal bit for bit, in either precision, for whole prompts,
portions beside decoded tokens and decode steps replayed from graphs."""
import numpy as np
import pytest
import torch

import helpers as H
from test_engine_gpu import TORCH, mixed_schedule

pytestmark = pytest.mark.gpu


def runner_for(folder, dtype, python_walk, monkeypatch, **kw):
    from allpaca_amd.engine.runner import ModelRunner
    from allpaca_amd.models import load_model
    if python_walk:
        monkeypatch.setenv("ALLPACA_AMD_PYTHON_WALK", "1")
    else:
        monkeypatch.delenv("ALLPACA_AMD_PYTHON_WALK", raising=False)
    cfg, model = load_model(folder, TORCH[dtype], "cuda:0")
    runner = ModelRunner(model, 16, 64, 8, **kw)
    assert (runner.native is None) == python_walk
    return cfg, runner


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_the_executor_gives_the_python_walks_bits(name, dtype, monkeypatch):
    from allpaca_amd.engine.batch import Entry
    folder = H.model_folder(name, dtype, True)
    lengths = {"A": [100, 2, 77, 40, 120, 33, 9], "B": [150, 2, 77, 40, 120, 33, 9], "C": [150, 2, 77, 40, 300, 33, 9]}[name]
    out = []
    for python_walk in (True, False):
        cfg, runner = runner_for(folder, dtype, python_walk, monkeypatch)
        toks = [H.random_tokens(cfg.vocab_size, n, seed=100 + i) for i, n in enumerate(lengths)]
        got = []
        for entries, ends in mixed_schedule(lengths, seed=11):
            batch = []
            for i, at, n in entries:
                if i not in runner.cache:
                    runner.admit(i)
                batch.append(Entry(i, toks[i][at:at + n], list(range(0, n, 2))))
            got.append(runner.step(batch).cpu().numpy())
            for i in ends:
                runner.release(i)
        out.append(got)
    for a, b in zip(*out):
        assert np.array_equal(a, b)


def test_real_widths_through_every_kind_of_product(monkeypatch):
    """Widths at which the bfloat16 path takes its MFMA kernels (tiled weights, the folded norm, q/k/v with rotation in
    the product, K in slices, the 128-row attention tiles): steps of 1, 8, 40, 200, 520 and 1,100 rows."""
    from allpaca_amd.engine.batch import Entry
    from allpaca_amd.weights import write_model_folder
    import os
    cfg = dict(H.TINY_B, hidden_size=1024, num_attention_heads=8, num_key_value_heads=2, head_dim=128,
               intermediate_size=2816, num_hidden_layers=2, vocab_size=4000, max_position_embeddings=4096,
               rope_scaling=None)
    folder = os.path.join(H.tmp_root(), "native_wide")
    if not os.path.isdir(folder):
        write_model_folder(folder, cfg, 5, torch.bfloat16)
    out = []
    for python_walk in (True, False):
        _, runner = runner_for(folder, "bfloat16", python_walk, monkeypatch)
        runner.cache  # pages: 64 x 16 = 1,024 positions in all is too few for this test's prompts
        from allpaca_amd.engine.runner import ModelRunner
        runner = ModelRunner(runner.model, 16, 400, 12)
        got = []
        rng = np.random.default_rng(3)
        for s, n in enumerate([1, 8, 40, 200, 520, 1100]):
            runner.admit(("p", s))
            toks = rng.integers(0, 4000, size=n).tolist()
            batch = [Entry(("p", s), toks, [n - 1])]
            # beside the prompt: every earlier request decodes a token
            batch += [Entry(("p", t), [int(rng.integers(0, 4000))], [0]) for t in range(s)]
            got.append(runner.step(batch).cpu().numpy())
        out.append(got)
    for a, b in zip(*out):
        assert np.array_equal(a, b)


def test_decode_graphs_on_the_executor(monkeypatch):
    from allpaca_amd.engine.batch import Entry
    folder = H.model_folder("B", "bfloat16", True)
    cfg, runner = runner_for(folder, "bfloat16", False, monkeypatch, use_graphs=True)
    _, eager = runner_for(folder, "bfloat16", False, monkeypatch, use_graphs=False)
    toks = [H.random_tokens(cfg.vocab_size, 60, seed=i) for i in range(3)]
    for r in (runner, eager):
        for i in range(3):
            r.admit(i)
            r.step([Entry(i, toks[i][:20 + i], [])])
    for t in range(30):
        batch = [Entry(i, [toks[i][20 + i + t]], [0]) for i in range(3)]
        a, b = runner.step(batch), eager.step(batch)
        assert torch.equal(a, b), f"decode step {t}"
    assert runner.graph_replays == 30
