"""The engine against the plain implementation, in float32 and in bfloat16, under
every cutting of the work: each request alone and whole; most of it in one step
and the last 32 tokens one by one; portions of changing size down to two tokens;
mixed batches of up to four live requests with so few pages that they are used
again; long decoding; the first tokens of a sequence."""
import numpy as np
import pytest
import torch

import helpers as H

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]
TORCH = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def make_runner(folder, dtype, page_tokens=16, num_pages=64, max_requests=8, max_positions=None, poison=False):
    from allpaca_amd.engine.runner import ModelRunner
    from allpaca_amd.models import load_model
    cfg, model = load_model(folder, TORCH[dtype], "cuda:0", max_positions=max_positions)
    return cfg, ModelRunner(model, page_tokens, num_pages, max_requests, poison_free_pages=poison)


def run_cut(runner, seq, tokens, cuts):
    """Feeds `tokens` of one request in portions `cuts`, asking for every row's logits."""
    from allpaca_amd.engine.batch import Entry
    runner.admit(seq)
    out, at = [], 0
    for n in cuts:
        lg = runner.step([Entry(seq, tokens[at:at + n], list(range(n)))])
        out.append(lg.float().cpu().numpy())
        at += n
    runner.release(seq)
    assert at == len(tokens)
    return np.concatenate(out, axis=0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C"])
@pytest.mark.parametrize("sharp", [False, True])
def test_whole_tail_and_portions(name, dtype, sharp):
    folder = H.model_folder(name, dtype, sharp)
    cfg, runner = make_runner(folder, dtype)
    lens = {"A": [1, 7, 16, 33, 100], "B": [2, 33, 150], "C": [5, 64, 129]}[name]
    for i, n in enumerate(lens):
        toks = H.random_tokens(cfg.vocab_size, n, seed=10 * i + 1)
        whole = run_cut(runner, "w", toks, H.cut_whole(n))
        H.check_logits(whole, folder, toks, dtype, f"{name} whole n={n}")
        tail = run_cut(runner, "t", toks, H.cut_tail_decoded(n))
        H.check_logits(tail, folder, toks, dtype, f"{name} tail-decoded n={n}")
        for s in range(2):
            cuts = H.cut_changing(n, seed=s)
            got = run_cut(runner, "c", toks, cuts)
            H.check_logits(got, folder, toks, dtype, f"{name} portions {cuts}")
        if dtype == "float32":
            # rows do not depend on the cutting at all: the products and the attention of a row
            # add in an order that its position alone fixes
            assert np.array_equal(whole, tail), f"{name} n={n}: whole and tail-decoded logits differ in bits"
    runner.cache.check()
    assert runner.cache.free_pages(0) == 64


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B"])
def test_first_tokens_and_page_sizes(name, dtype):
    """The first tokens of a sequence (positions 0, 1, 2), and the same logits for any page size."""
    folder = H.model_folder(name, dtype, True)
    toks = None
    for page_tokens in (1, 2, 16, 64):
        cfg, runner = make_runner(folder, dtype, page_tokens=page_tokens, num_pages=80)
        toks = toks or H.random_tokens(cfg.vocab_size, 40, seed=3)
        got = run_cut(runner, "p", toks, [1, 1, 1, 2, 35])
        H.check_logits(got, folder, toks, dtype, f"{name} page_tokens={page_tokens}")


def mixed_schedule(lengths, seed, live_max=4):
    """Steps of a mixed batch: requests start at different times, advance by portions of changing
    size or single tokens, some pause for a step, and end; at most `live_max` are live."""
    rng = np.random.default_rng(seed)
    todo = list(range(len(lengths)))
    done_at = {i: 0 for i in todo}
    live, steps = [], []
    while todo or live:
        while todo and len(live) < live_max and (not live or rng.random() < 0.6):
            live.append(todo.pop(0))
        entries, ends = [], []
        for i in list(live):
            left = lengths[i] - done_at[i]
            if len(live) > 1 and rng.random() < 0.15:
                continue  # left out of this step, goes on later
            mode = rng.random()
            n = 1 if mode < 0.45 else int(rng.choice([2, 2, 3, 5, 8, 13, 21, 40]))
            n = min(n, left)
            entries.append((i, done_at[i], n))
            done_at[i] += n
            if done_at[i] == lengths[i]:
                ends.append(i)
                live.remove(i)
        if entries:
            steps.append((entries, ends))
    return steps


def run_mixed(name, dtype, poison):
    """The mixed schedule of test_mixed_batches_with_page_reuse; returns the runner, the tokens and every request's
    logits.  `poison`: what free pages are filled with, at the start and whenever one comes back (False: nothing)."""
    from allpaca_amd.engine.batch import Entry
    folder = H.model_folder(name, dtype, True)
    lengths = {"A": [33, 100, 16, 7, 64, 1, 90, 50], "B": [150, 2, 77, 40, 120, 33, 9], "C": [129, 64, 5, 200, 31, 90]}[name]
    # pages for four live requests of the longest kind only: finished requests' pages must be used again
    page_tokens = 16
    worst = sorted(lengths)[-4:]
    num_pages = sum(-(-n // page_tokens) for n in worst)
    cfg, runner = make_runner(folder, dtype, page_tokens=page_tokens, num_pages=num_pages, poison=poison)
    toks = [H.random_tokens(cfg.vocab_size, n, seed=100 + i) for i, n in enumerate(lengths)]
    got = {i: [] for i in range(len(lengths))}
    for entries, ends in mixed_schedule(lengths, seed=7):
        batch = []
        for i, at, n in entries:
            if i not in runner.cache:
                runner.admit(i)
            batch.append(Entry(i, toks[i][at:at + n], list(range(n))))
        lg = runner.step(batch).float().cpu().numpy()
        row = 0
        for i, at, n in entries:
            got[i].append(lg[row:row + n])
            row += n
        for i in ends:
            runner.release(i)
        runner.cache.check()
    assert runner.cache.paged_groups[0].pool.allocations > num_pages, "the schedule did not reuse pages"
    assert runner.cache.free_pages(0) == num_pages
    return folder, runner, toks, [np.concatenate(got[i]) for i in range(len(lengths))]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_mixed_batches_with_page_reuse(name, dtype):
    # free pages are filled with 1e30, at the start and whenever one comes back: a key or value read from a page
    # before its new owner wrote it would show in the logits
    folder, runner, toks, got = run_mixed(name, dtype, True)
    n = runner.cache.paged_groups[0].pool.num_pages
    assert bool((runner.storage.paged[0][:, :n].float() > 1e29).all()), "pages that came back are not filled"
    for i, t in enumerate(toks):
        H.check_logits(got[i], folder, t, dtype, f"{name} mixed request {i}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_nan_in_free_pages_changes_no_bit(name, dtype):
    """A page that comes back may hold anything, NaN too (a request whose activations blew up), and a slot beyond a
    row's last key gets a weight of 0 in the value product: 0 x NaN would be NaN, for this request and, through
    what it writes, for the next owner of its pages.  With NaN in every free page the logits are the same, bit for
    bit, as with pages that hold zeros."""
    _, _, _, clean = run_mixed(name, dtype, False)
    _, runner, _, dirty = run_mixed(name, dtype, float("nan"))
    n = runner.cache.paged_groups[0].pool.num_pages
    assert bool(torch.isnan(runner.storage.paged[0][:, :n].float()).all()), "pages that came back are not filled"
    for i, (a, b) in enumerate(zip(clean, dirty)):
        assert np.isfinite(b).all(), f"{name} request {i}: non-finite logits with NaN in free pages"
        assert np.array_equal(a, b), f"{name} request {i}: NaN in free pages changed the logits"


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding(dtype):
    """A short prompt and 200 tokens decoded one by one, across many page edges."""
    folder = H.model_folder("B", dtype, True)
    cfg, runner = make_runner(folder, dtype, page_tokens=16, num_pages=20)
    toks = H.random_tokens(cfg.vocab_size, 230, seed=5)
    got = run_cut(runner, "d", toks, [30] + [1] * 200)
    H.check_logits(got, folder, toks, dtype, "long decoding")


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_far_key_is_found(dtype):
    """One early token is made to match the last query exactly with a large score in every head of layer 0;
    the result must follow that token's value whatever stands between."""
    import plain_llama as P
    from allpaca_amd.weights import write_model_folder
    import os
    cfg = dict(H.TINY_B, num_hidden_layers=1, rope_scaling=None)
    D, Hh, Hk, d = 192, 6, 2, 32
    wq = torch.zeros(Hh * d, D)
    wk = torch.zeros(Hk * d, D)
    # keys answer to coordinate 0 of the normed input and queries to coordinate 1, both through the slowest
    # rotation pair (index d/2 - 1 turns by < 1e-3 rad over 300 positions).  Token 7 alone carries coordinate 0
    # and token 9 alone carries coordinate 1: a row holding token 9 scores ~2000 on rows holding token 7 and
    # exactly 0 on every other row, itself included.
    for h in range(Hh):
        wq[h * d + d // 2 - 1, 1] = 8.0
    for h in range(Hk):
        wk[h * d + d // 2 - 1, 0] = 8.0
    emb = torch.randn(1000, D, generator=torch.Generator().manual_seed(0)) * 0.02
    emb[:, 0] = 0.0
    emb[:, 1] = 0.0
    emb[7, 0] = 3.0      # the marked token
    emb[9, 1] = 3.0      # the asking token
    path = os.path.join(H.tmp_root(), f"farkey_{dtype}")
    write_model_folder(path, cfg, 3, TORCH[dtype], overrides={
        "model.layers.0.self_attn.q_proj.weight": wq, "model.layers.0.self_attn.k_proj.weight": wk,
        "model.embed_tokens.weight": emb})
    toks = [t if t not in (7, 9) else 8 for t in H.random_tokens(1000, 250, seed=1)]
    toks[19] = 7
    toks[-1] = 9
    _, runner = make_runner(path, dtype)
    want = H.oracle_logits(path, toks)
    for cuts in ([250], [249, 1], [17, 3, 100, 2, 127, 1]):
        got = run_cut(runner, "f", toks, cuts)
        H.check_logits(got, path, toks, dtype, f"far key, cuts {cuts}")
    without = list(toks)
    without[19] = 8  # no marked token: the logits at the end are far from the ones found above
    assert np.abs(H.oracle_logits(path, without)[-1] - want[-1]).max() > 0.1


def test_widths_of_an_8b_model_against_the_plain_implementation_and_between_the_paths():
    """The tiny configurations do not reach the code paths that sizes choose (bands per block, waves per block,
    K in slices or whole, the fused product for q, k, v with d = 128, the llama3 table of a real model): two layers
    at the widths of an 8B model (hidden 4096, 32 heads over 8 of 128, feed-forward 14336; a small vocabulary),
    weights made on the GPU, the same bfloat16 values in both runs.  A whole portion, a mixed step, decode steps
    (replayed graphs) and a portion behind them are compared with the plain implementation on the same values, in
    32-bit and in bfloat16; further steps (42 decode rows, 600 and 1,100 rows) between the two paths: every row's
    logits are within the storage noise of two layers of the 32-bit path's, and no path is further off than the
    others."""
    import plain_llama as P
    from allpaca_amd.config import preset
    from allpaca_amd.engine.batch import Entry
    from allpaca_amd.engine.runner import ModelRunner
    from allpaca_amd.models import DecoderModel, describe_model
    from allpaca_amd.parts import Runtime
    from allpaca_amd.weights import random_tensors
    V = 8200
    cfg_json = dict(preset("llama-3.1-8b"), num_hidden_layers=2, vocab_size=V)
    sharpen = (3.0 / (0.02 ** 2 * cfg_json["hidden_size"])) ** 0.5      # scores of deviation ~3, as in helpers.model_folder
    plain_weights = {}

    def runner(dtype):
        _, _, spec = describe_model(cfg_json)
        model = DecoderModel(spec)
        tensors = {}
        for name, ps in model.param_specs().items():
            for k, v in random_tensors({name: ps}, 0, torch.bfloat16, 0.02, 0.0, device="cuda:0").items():
                if k.endswith("q_proj.weight") or k.endswith("k_proj.weight"):
                    v = (v.float() * sharpen).to(torch.bfloat16)
                tensors[k] = v if dtype == torch.bfloat16 else v.float()
                if k not in plain_weights:
                    plain_weights[k] = v.float().cpu().numpy()           # the plain side widens them itself
        model.bind(tensors, Runtime(torch.device("cuda:0"), dtype, 1280))
        return ModelRunner(model, 16, 192, 48, use_graphs=True)

    toks = H.random_tokens(V, 420, seed=5)
    rows = {}
    fed = {}      # request -> its tokens so far
    for dtype in (torch.float32, torch.bfloat16):
        r = runner(dtype)
        fed.clear()
        out = []

        def step(what, entries):
            where = []
            for e in entries:
                have = fed.setdefault(e.seq, [])
                where += [(e.seq, len(have) + w) for w in e.want]
                have += list(e.tokens)
            out.append((what, r.step(entries).float().cpu().numpy().astype(np.float64), where))

        r.admit("a")
        r.admit("b")
        step("whole portion", [Entry("a", toks[:300], list(range(300)))])
        step("mixed step", [Entry("a", toks[300:340], list(range(40))), Entry("b", toks[:17], list(range(17)))])
        for j in range(6):
            step("decode step", [Entry("a", [toks[340 + j]], [0]), Entry("b", [toks[17 + j]], [0])])
        step("portion behind", [Entry("a", toks[346:400], [0, 53]), Entry("b", toks[23:24], [0])])
        assert r.graph_replays == 6
        # 40 more requests: a mixed step of 160 rows, two decode steps of 42 rows (the tiled product with K in slices
        # and the folded norm in its finishing kernel), and a portion of 600 rows (K in slices for the narrow matrices)
        more = [f"m{i}" for i in range(40)]
        for m in more:
            r.admit(m)
        step("many short prompts", [Entry(m, toks[i:i + 4], [3]) for i, m in enumerate(more)])
        for j in range(2):
            step("decode step of 42 rows", [Entry("a", [toks[400 + j]], [0]), Entry("b", [toks[24 + j]], [0])]
                 + [Entry(m, [toks[i + 4 + j]], [0]) for i, m in enumerate(more)])
        r.release("a")
        r.admit("c")
        step("portion of 600 rows", [Entry("c", (toks * 2)[:600], [0, 299, 599])])
        # 1,100 rows: SwiGLU on the tile of 256 rows for most of its columns and on the tile of 128 rows for the rest
        r.release("c")
        r.admit("d")
        step("portion of 1,100 rows", [Entry("d", (toks * 3)[:1100], [0, 550, 1099])])
        rows[dtype] = out
        del r
        torch.cuda.empty_cache()
    # against the plain implementation: requests a and b (402 and 26 tokens), every row that was asked for
    exact = {s: P.llama_forward(cfg_json, plain_weights, fed[s]) for s in ("a", "b")}
    noisy = {s: P.llama_forward(cfg_json, plain_weights, fed[s], store=P.round_bf16) for s in ("a", "b")}
    for dtype, name in ((torch.float32, "float32"), (torch.bfloat16, "bfloat16")):
        for what, lg, where in rows[dtype]:
            keep = [i for i, (s, _) in enumerate(where) if s in exact]
            if not keep:
                continue
            want = np.stack([exact[where[i][0]][where[i][1]] for i in keep])
            noise = np.stack([noisy[where[i][0]][where[i][1]] for i in keep])
            if name == "float32":
                # the bound of the tiny models (2e-5 on logits of magnitude 0.3), relative to these logits' size
                assert np.abs(lg[keep] - want).max() <= H.F32_ATOL / 0.3 * np.abs(want).max(), what
            else:
                H.assert_close(lg[keep], want, name, f"8B widths, {what}", noise)
    errs = []
    for (what, a, _), (_, b, _) in zip(rows[torch.float32], rows[torch.bfloat16]):
        e = np.sqrt(((a - b) ** 2).mean(axis=1)) / np.sqrt((a ** 2).mean(axis=1))
        errs.append((what, float(e.max()), float(e.mean())))
    # measured: 0.016 on average, 0.021 at most, the same on every path
    worst = max(e for _, e, _ in errs)
    mean = float(np.mean([m for _, _, m in errs]))
    assert worst < 0.03 and worst < 2.0 * mean, errs


@pytest.mark.parametrize("widths", ["llama-3.1-8b", "llama-3.2-1b"])
def test_a_long_prompt_at_the_widths_of_a_real_model_in_portions_of_512_and_128(widths):
    """Two layers at the widths of Llama-3.1-8B (heads of 128) and of Llama-3.2-1B (heads of 64, the head tied to the
    embedding), a prompt of 4,500 tokens: in steps of 2,048 rows (a block of the
    attention kernel per tile of 128 rows and head, but for the last step's 404 rows), in steps of 512 and of 128 rows
    (from 4,096 keys on the keys of a tile are cut into ranges for several blocks and a second kernel adds them) and
    in 32-bit: the logits of the rows asked for are those of the plain implementation on the same values in 32-bit,
    and within the storage noise of two layers of them in bfloat16, on every path alike."""
    from allpaca_amd.config import preset
    from allpaca_amd.engine.batch import Entry
    from allpaca_amd.engine.runner import ModelRunner
    from allpaca_amd.kernels import tuned
    from allpaca_amd.models import DecoderModel, describe_model
    from allpaca_amd.parts import Runtime
    from allpaca_amd.weights import random_tensors
    import plain_llama as P
    V, T = 8200, 4500
    cfg_json = dict(preset(widths), num_hidden_layers=2, vocab_size=V)
    sharpen = (3.0 / (0.02 ** 2 * cfg_json["hidden_size"])) ** 0.5
    plain_weights = {}

    def runner(dtype):
        _, _, spec = describe_model(cfg_json)
        model = DecoderModel(spec)
        tensors = {}
        for name, ps in model.param_specs().items():
            for k, v in random_tensors({name: ps}, 0, torch.bfloat16, 0.02, 0.0, device="cuda:0").items():
                if k.endswith("q_proj.weight") or k.endswith("k_proj.weight"):
                    v = (v.float() * sharpen).to(torch.bfloat16)
                tensors[k] = v if dtype == torch.bfloat16 else v.float()
                if k not in plain_weights:
                    plain_weights[k] = v.float().cpu().numpy()
        model.bind(tensors, Runtime(torch.device("cuda:0"), dtype, T + 64))
        return ModelRunner(model, 16, (T + 64) // 16 + 8, 4, use_graphs=False)

    toks = H.random_tokens(V, T, seed=11)
    asked = [4100, 4223, 4351, T - 1]          # positions whose logits are compared
    n_heads = cfg_json["num_attention_heads"]

    def run(dtype, portion, seen):
        r = runner(dtype)
        forward = r.forward
        # into how many ranges the attention kernel cuts the keys of this step's tiles (the executor's rule is the
        # wrappers' own: tests/test_dispatch_rules.py)
        r.forward = lambda info: seen.append(tuned._key_splits(info, n_heads, 0)) or forward(info)
        r.admit("p")
        got, at = {}, 0
        while at < T:
            n = min(portion, T - at)
            want = [p - at for p in asked if at <= p < at + n]
            lg = r.step([Entry("p", toks[at:at + n], want)])
            if want:
                for w, row in zip(want, lg.float().cpu().numpy().astype(np.float64)):
                    got[at + w] = row
            at += n
        del r
        torch.cuda.empty_cache()
        return np.stack([got[p] for p in asked])

    exact = run(torch.float32, 2048, [])
    # the 32-bit path against the plain implementation on the same values (the bound of the tiny models, 2e-5 on
    # logits of magnitude 0.3, relative to these logits' size)
    plain = P.llama_forward(cfg_json, plain_weights, toks)[asked]
    assert np.abs(exact - plain).max() <= H.F32_ATOL / 0.3 * np.abs(plain).max()
    cut = {}
    for portion in (2048, 512, 128):
        seen = []
        cut[portion] = run(torch.bfloat16, portion, seen)
        assert max(seen) > 1, portion       # (also with 2,048: the last step has the 404 rows that are left)
    errs = {p: np.sqrt(((lg - plain) ** 2).mean(axis=1)) / np.sqrt((plain ** 2).mean(axis=1)) for p, lg in cut.items()}
    worst = max(float(e.max()) for e in errs.values())
    mean = float(np.mean([e.mean() for e in errs.values()]))
    # (the widths test above measures 0.016 on average and 0.021 at most between the two precisions)
    assert worst < 0.03 and worst < 2.0 * mean, errs


@pytest.mark.parametrize("stored,run", [("float32", "bfloat16"), ("bfloat16", "float32")])
def test_a_model_stored_in_one_precision_runs_in_the_other(stored, run):
    """Matrices stored in 32-bit stay so in a bfloat16 run (activations are bfloat16, the products take the plain
    kernels); matrices stored in bfloat16 are widened for a 32-bit run.  Logits against the plain implementation on
    the folder's own values, whole and cut."""
    for name in ("A", "B"):
        folder = H.model_folder(name, stored, True)
        cfg, runner = make_runner(folder, run)
        toks = H.random_tokens(cfg.vocab_size, 70, seed=3)
        for cuts in (H.cut_whole(70), H.cut_tail_decoded(70), H.cut_changing(70, 2)):
            got = run_cut(runner, "x", toks, cuts)
            H.check_logits(got, folder, toks, run, f"{name} stored {stored}, run {run}, {cuts[:4]}")
