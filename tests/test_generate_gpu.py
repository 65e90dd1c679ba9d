"""Generation through the entry points: greedy and sampled tokens against the plain
implementation, concurrency against solo runs, preemption, the command line and
the trace replay program."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import helpers as H
import plain_llama as P

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def engine_for(folder, dtype="float32", **opts):
    from allpaca_amd.engine import Engine
    base = dict(dtype=dtype, max_tokens=1024, max_active_requests=8, use_graphs=False)
    base.update(opts)
    return Engine(folder, **base)


def params(**kw):
    from allpaca_amd.sampling import GenerationParams
    return GenerationParams(**kw)


def test_greedy_generation_equals_the_plain_implementation():
    """Tiny A: prompts of 1, 7, 16 and 33 tokens, 16 greedy tokens each, alone and as chunked mixed batches."""
    folder = H.model_folder("A", "float32", True)
    cfg, w = H.oracle(folder)
    prompts = [H.random_tokens(256, n, seed=n) for n in (1, 7, 16, 33)]
    want = [P.greedy_generate(cfg, w, p, 16) for p in prompts]
    eng = engine_for(folder)
    for p, wnt in zip(prompts, want):
        out = eng.generate([p], params(max_tokens=16, temperature=0.0))[0]
        assert out.token_ids == wnt and out.finish_reason == "length" and out.prompt_tokens == len(p)
    eng = engine_for(folder, chunk_tokens=8, max_batch_tokens=12)
    outs = eng.generate(prompts, params(max_tokens=16, temperature=0.0))
    assert [o.token_ids for o in outs] == want
    assert eng.stats["steps"] < sum(len(p) + 16 for p in prompts)   # prompts ran in portions, not token by token


def test_sampled_generation_equals_the_plain_sampler():
    """Tiny B: six prompts of 2 to 150 tokens, temperature 0.8 (top-k 40, top-p 0.95), 24 tokens each:
    every token is what the plain sampler draws from the plain logits of the same context with the same
    uniform number."""
    from allpaca_amd.sampling.sampler import uniform_for
    folder = H.model_folder("B", "float32", True)
    cfg, w = H.oracle(folder)
    prompts = [H.random_tokens(1000, n, seed=n) for n in (2, 9, 31, 64, 100, 150)]
    eng = engine_for(folder, chunk_tokens=32, max_batch_tokens=48)
    pr = [params(max_tokens=24, temperature=0.8, seed=7 + i) for i in range(len(prompts))]
    outs = eng.generate(prompts, pr)
    for i, (p, o) in enumerate(zip(prompts, outs)):
        assert len(o.token_ids) == 24
        toks = list(p)
        for j, t in enumerate(o.token_ids):
            if j % 6 == 0:   # every sixth token is checked against the oracle (each check is a whole forward)
                lg = P.llama_forward(cfg, w, toks)[-1]
                assert t == P.sample(lg, 0.8, 40, 0.95, uniform_for(7 + i, j)), f"prompt {i} token {j}"
            toks.append(t)
    assert len({tuple(o.token_ids) for o in outs}) == len(outs)


def test_same_seed_same_tokens_under_any_batching_and_stop_ids():
    folder = H.model_folder("B", "float32", True)
    prompts = [H.random_tokens(1000, n, seed=50 + n) for n in (3, 40, 77, 12, 130)]
    pr = [params(max_tokens=12, temperature=0.9, top_k=0, top_p=1.0, seed=3),
          params(max_tokens=12, temperature=0.0),
          params(max_tokens=12, temperature=0.7, top_k=5, seed=11),
          params(max_tokens=12, temperature=1.3, top_k=0, top_p=0.6, seed=5),
          params(max_tokens=12, temperature=0.8)]
    solo = [engine_for(folder).generate([p], q)[0].token_ids for p, q in zip(prompts, pr)]
    together = engine_for(folder, chunk_tokens=16, max_batch_tokens=24).generate(prompts, pr)
    assert [o.token_ids for o in together] == solo        # crates/allpaca-core/tests/hip_runtime.rs:8149-8176 in spirit
    stop = solo[1][4]
    first = solo[1].index(stop)
    out = engine_for(folder).generate([prompts[1]], params(max_tokens=12, temperature=0.0, stop_token_ids=[stop]))[0]
    assert out.token_ids == solo[1][: first + 1] and out.finish_reason == "stop"   # the stop token is emitted


def test_sampled_tokens_are_the_same_with_steps_queued_ahead():
    """With graphs the engine queues a step before the tokens of the one before have reached the host; the index
    of a request's random number then counts the token that is still on its way."""
    folder = H.model_folder("B", "float32", True)
    prompts = [H.random_tokens(1000, n, seed=90 + n) for n in (3, 40, 12, 25)]
    pr = [params(max_tokens=20, temperature=0.9, top_k=0, top_p=1.0, seed=3),
          params(max_tokens=14, temperature=0.0),
          params(max_tokens=20, temperature=0.7, top_k=5, seed=11),
          params(max_tokens=9, temperature=1.3, top_k=0, top_p=0.6, seed=5)]
    eager = engine_for(folder).generate(prompts, pr)
    eng = engine_for(folder, use_graphs=True)
    queued = eng.generate(prompts, pr)
    assert [o.token_ids for o in queued] == [o.token_ids for o in eager]
    assert eng.runner.graph_replays > 10


def test_preemption_gives_the_same_tokens():
    folder = H.model_folder("A", "float32", True)
    prompts = [H.random_tokens(256, n, seed=70 + n) for n in (30, 25, 28)]
    pr = params(max_tokens=40, temperature=0.8, seed=1)
    solo = [engine_for(folder).generate([p], pr)[0].token_ids for p in prompts]
    # 3 requests grow to ~70 tokens = 5 pages each; 11 pages cannot hold them all: someone must give way
    eng = engine_for(folder, num_pages=11, max_active_requests=3)
    outs = eng.generate(prompts, pr)
    assert eng.stats["preemptions"] > 0
    assert [o.token_ids for o in outs] == solo
    assert eng.runner.cache.free_pages(0) == 11
    eng.runner.cache.check()


def test_stream_and_low_level_calls():
    folder = H.model_folder("A", "float32")
    eng = engine_for(folder)
    p = H.random_tokens(256, 9, seed=1)
    evs = list(eng.generate_stream(p, params(max_tokens=5, temperature=0.0)))
    assert [e.finish_reason for e in evs] == [None] * 4 + ["length"] and all(e.prompt_tokens == 9 for e in evs)
    rid = eng.begin_request(p, params(max_tokens=5, temperature=0.0))
    got = []
    while eng.has_unfinished():
        got += [e.token_id for e in eng.poll() if e.request_id == rid]
    assert got == [e.token_id for e in evs]
    from allpaca_amd.engine import RequestTooLarge
    with pytest.raises(ValueError):
        eng.add_request([256])                       # outside the vocabulary
    small = engine_for(folder, num_pages=2)
    with pytest.raises((RequestTooLarge, ValueError)):
        small.add_request(p, params(max_tokens=60))


def test_command_line_generate():
    folder = H.model_folder("A", "float32", True)
    cfg, w = H.oracle(folder)
    p1, p2 = H.random_tokens(256, 5, seed=1), H.random_tokens(256, 11, seed=2)
    spec = ",".join(map(str, p1)) + ";" + ",".join(map(str, p2))
    cmd = [sys.executable, os.path.join(ROOT, "bin", "allpaca-amd"), "generate", "--model", folder, "--dtype", "fp32",
           "--prompt-tokens", spec, "--max-tokens", "6", "--temperature", "0", "--json"]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=280)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [json.loads(ln) for ln in r.stdout.strip().splitlines()]
    assert [ln["token_ids"] for ln in lines] == [P.greedy_generate(cfg, w, p, 6) for p in (p1, p2)]
    assert all(0 <= ln["queue_ms"] <= ln["ttft_ms"] and ln["itl_ms"] > 0 for ln in lines)   # times per request
    r = subprocess.run(cmd[:2] + ["generate", "--synthetic", "--cpu-only", "--prompt-tokens", "1"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 2 and ("no CPU path" in r.stderr or "not available" in r.stderr), (r.returncode, r.stderr[-500:])


def replay(folder, dtype, steps, max_tokens, out_dir, page_tokens=16):
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
           "--out", out_dir, "--max-tokens", str(max_tokens), "--page-tokens", str(page_tokens),
           "--poison-free-pages"]     # free pages hold 1e30: a read of a page before its owner wrote it would show
    text = "".join(json.dumps(s) + "\n" for s in steps)
    r = subprocess.run(cmd, input=text, capture_output=True, text=True, timeout=280)
    assert r.returncode == 0, r.stderr[-3000:]
    assert r.stdout.split() == [w for s in steps for w in ("done", str(s["step"]))]
    return r


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(dtype, tmp_path):
    """The replay program, as a user runs it: the same requests whole, with the last 32 tokens decoded one by
    one, and mixed with other requests so that pages are used again."""
    folder = H.model_folder("B", dtype, True)
    V = 1000
    lens = [70, 150, 33, 100, 64]
    toks = {f"r{i}": H.random_tokens(V, n, seed=200 + i) for i, n in enumerate(lens)}
    # whole
    steps = [dict(step=i, entries=[dict(id=k, tokens=t, want=list(range(len(t))))], end=[k])
             for i, (k, t) in enumerate(toks.items())]
    out = str(tmp_path / "whole")
    replay(folder, dtype, steps, 192, out)
    for i, (k, t) in enumerate(toks.items()):
        got = np.fromfile(os.path.join(out, f"{i}.f32"), dtype="<f4").reshape(len(t), V)
        H.check_logits(got, folder, t, dtype, f"trace whole {k}")
    # tail decoded: logits wanted only at the last prompt row and at the decoded ones; a step without `want`
    k, t = "r1", toks["r1"]
    steps = [dict(step=0, entries=[dict(id=k, tokens=t[:60], want=[])], end=[]),
             dict(step=1, entries=[dict(id=k, tokens=t[60:118], want=[57])], end=[])]
    steps += [dict(step=2 + j, entries=[dict(id=k, tokens=[t[118 + j]], want=[0])], end=[k] if j == 31 else [])
              for j in range(32)]
    out = str(tmp_path / "tail")
    replay(folder, dtype, steps, 192, out)
    assert not os.path.exists(os.path.join(out, "0.f32"))
    rows = [np.fromfile(os.path.join(out, f"{s}.f32"), dtype="<f4").reshape(1, V) for s in range(1, 34)]
    want_rows = list(range(117, 150))
    noise = H.oracle_logits_bf16_storage(folder, t)[want_rows] if dtype == "bfloat16" else None
    H.assert_close(np.concatenate(rows), H.oracle_logits(folder, t)[want_rows], dtype, "trace tail", noise)
    # mixed, four live at most, pool of 4 x 64-rounded tokens of the smaller requests: pages are used again
    import test_engine_gpu as E
    sched = E.mixed_schedule(lens, seed=3)
    steps, got = [], {k: [] for k in toks}
    keys = list(toks)
    for si, (entries, ends) in enumerate(sched):
        steps.append(dict(step=si, entries=[dict(id=keys[i], tokens=toks[keys[i]][at:at + n], want=list(range(n)))
                                            for i, at, n in entries], end=[keys[i] for i in ends]))
    out = str(tmp_path / "mixed")
    live_budget = sum(sorted(-(-n // 64) * 64 for n in lens)[-4:])
    replay(folder, dtype, steps, live_budget, out)
    for si, (entries, ends) in enumerate(sched):
        arr = np.fromfile(os.path.join(out, f"{si}.f32"), dtype="<f4").reshape(-1, V)
        row = 0
        for i, at, n in entries:
            got[keys[i]].append(arr[row:row + n])
            row += n
        assert row == arr.shape[0]
    for k, t in toks.items():
        H.check_logits(np.concatenate(got[k]), folder, t, dtype, f"trace mixed {k}")


def test_trace_run_goes_past_the_position_limit_of_config_json(tmp_path):
    """Tiny A names 128 positions; the replay of given tokens runs 200 (the formulas hold at any position and the
    reference does not read that key), as the plain implementation does."""
    folder = H.model_folder("A", "float32", True)
    t = H.random_tokens(256, 200, seed=77)
    # wanted places in any order, one of them twice: the rows come in the order asked for
    steps = [dict(step=0, entries=[dict(id="a", tokens=t[:150], want=[149, 100, 149])], end=[])]
    steps += [dict(step=1 + j, entries=[dict(id="a", tokens=[t[150 + j]], want=[0])], end=[]) for j in range(50)]
    out = str(tmp_path / "past")
    replay(folder, "float32", steps, 256, out)
    rows = [np.fromfile(os.path.join(out, f"{s}.f32"), dtype="<f4").reshape(-1, 256) for s in range(51)]
    H.assert_close(np.concatenate(rows), H.oracle_logits(folder, t)[[149, 100] + list(range(149, 200))], "float32",
                   "past the limit")


def test_trace_run_with_large_pages_and_many_live_requests(tmp_path):
    """Ten live requests of one to three tokens with pages of 128 positions: --max-tokens counts each request as 64
    tokens (640), and every one of them still needs a page of its own."""
    folder = H.model_folder("A", "float32", True)
    toks = {f"q{i}": H.random_tokens(256, 1 + i % 3, seed=400 + i) for i in range(10)}
    steps = [dict(step=0, entries=[dict(id=k, tokens=t[:1], want=[0]) for k, t in toks.items()], end=[]),
             dict(step=1, entries=[dict(id=k, tokens=t[1:], want=list(range(len(t) - 1))) for k, t in toks.items()
                                   if len(t) > 1], end=list(toks))]
    out = str(tmp_path / "many")
    replay(folder, "float32", steps, 640, out, page_tokens=128)
    first = np.fromfile(os.path.join(out, "0.f32"), dtype="<f4").reshape(10, 256)
    rest = np.fromfile(os.path.join(out, "1.f32"), dtype="<f4").reshape(-1, 256)
    row = 0
    for i, (k, t) in enumerate(toks.items()):
        got = [first[i:i + 1]]
        if len(t) > 1:
            got.append(rest[row:row + len(t) - 1])
            row += len(t) - 1
        H.check_logits(np.concatenate(got), folder, t, "float32", f"trace many {k}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_graph_replays_equal_eager_steps(dtype):
    """Decode-only steps replayed as HIP graphs give the logits of the same steps run eagerly: several replays of
    each graph, with eager prefill work, other graphs and synchronisations between them, growing contexts, changing
    numbers of live requests (so rows are padded) and page edges."""
    from allpaca_amd.engine.batch import Entry
    from allpaca_amd.engine.runner import ModelRunner
    from allpaca_amd.models import load_model
    folder = H.model_folder("B", dtype, True)
    tdt = torch.float32 if dtype == "float32" else torch.bfloat16
    cfg, model = load_model(folder, tdt, "cuda:0")
    runs = {}
    for graphs in (False, True):
        runner = ModelRunner(model, 16, 40, 8, use_graphs=graphs)
        toks = {i: H.random_tokens(1000, 90, seed=300 + i) for i in range(3)}
        out = []
        at = {}
        for i, n0 in ((0, 5), (1, 30)):
            runner.admit(i)
            runner.step([Entry(i, toks[i][:n0], [])])
            at[i] = n0
        for s in range(40):
            if s == 7:                                   # a third request joins: eager prefill between replays
                runner.admit(2)
                runner.step([Entry(2, toks[2][:17], [])])
                at[2] = 17
            if s == 25:                                  # and one leaves: three rows -> two of a four-row graph
                runner.release(0)
                del at[0]
            batch = [Entry(i, [toks[i][p]], [0]) for i, p in sorted(at.items())]
            lg = runner.step(batch)
            out.append(lg.float().cpu().numpy())
            for i in at:
                at[i] += 1
        runs[graphs] = out
        if graphs:
            assert runner.graph_replays == 40 and len(runner.graphs) >= 2
    for a, b in zip(runs[False], runs[True]):
        if dtype == "float32":
            assert np.array_equal(a, b)
        else:
            # same kernels, but the number of key ranges a row is split into follows the graph's size
            assert np.abs(a - b).max() <= 2.0 ** -7 * np.abs(a).max()
    # and against the oracle
    i, upto = 1, 30 + 40
    toks1 = H.random_tokens(1000, 90, seed=301)
    got = np.concatenate([r[1 if k < 25 else 0][None] for k, r in enumerate(runs[True])])
    want_rows = list(range(30, 70))
    noise = H.oracle_logits_bf16_storage(folder, toks1[:upto])[want_rows] if dtype == "bfloat16" else None
    H.assert_close(got, H.oracle_logits(folder, toks1[:upto])[want_rows], dtype, "graph decode", noise)


def test_graphs_of_nine_to_sixteen_rows():
    """Decode steps of 9 to 16 requests are replayed from a graph of the next even number of rows (a padding row costs
    the streaming products what a live one does): 11 requests, then 9 when two have left, against eager steps and
    against the plain implementation; and the buckets that `capture_decode_graphs` makes for up to 13 requests."""
    from allpaca_amd.engine.batch import Entry
    from allpaca_amd.engine.runner import ModelRunner
    from allpaca_amd.models import load_model
    assert [ModelRunner._row_bucket(n) for n in (1, 2, 3, 5, 8, 9, 10, 11, 15, 16, 17, 33)] == \
        [1, 2, 4, 8, 8, 10, 10, 12, 16, 16, 32, 64]
    folder = H.model_folder("B", "float32", True)
    cfg, model = load_model(folder, torch.float32, "cuda:0")
    runs = {}
    for graphs in (False, True):
        runner = ModelRunner(model, 16, 96, 16, use_graphs=graphs)
        toks = {i: H.random_tokens(1000, 40, seed=500 + i) for i in range(11)}
        at = {}
        for i in range(11):
            runner.admit(i)
            runner.step([Entry(i, toks[i][:3 + i], [])])
            at[i] = 3 + i
        out = []
        for s in range(12):
            if s == 6:
                for i in (2, 7):
                    runner.release(i)
                    del at[i]
            out.append(runner.step([Entry(i, [toks[i][p]], [0]) for i, p in sorted(at.items())]).float().cpu().numpy())
            for i in at:
                at[i] += 1
        runs[graphs] = out
        if graphs:
            assert runner.graph_replays == 12 and {k[0] for k in runner.graphs} == {12, 10}
            assert runner.capture_decode_graphs(13, 64) > 0
            assert {k[0] for k in runner.graphs} == {1, 2, 4, 8, 10, 12, 14}
    for a, b in zip(runs[False], runs[True]):
        assert np.array_equal(a, b)
    got = np.concatenate([r[-1][None] for r in runs[True]])          # request 10: its tokens 13 .. 24
    H.assert_close(got, H.oracle_logits(folder, H.random_tokens(1000, 40, seed=510)[:25])[13:25], "float32", "graphs of 12 and 10 rows")


def test_generation_with_graphs_equals_the_plain_implementation():
    folder = H.model_folder("A", "float32", True)
    cfg, w = H.oracle(folder)
    prompts = [H.random_tokens(256, n, seed=n) for n in (1, 7, 16, 33)]
    want = [P.greedy_generate(cfg, w, p, 16) for p in prompts]
    eng = engine_for(folder, use_graphs=True, chunk_tokens=8, max_batch_tokens=12)
    outs = eng.generate(prompts, params(max_tokens=16, temperature=0.0))
    assert [o.token_ids for o in outs] == want
    assert eng.runner.graph_replays > 0


def test_graphs_captured_before_serving_are_the_ones_generation_asks_for():
    """`warm_up` captures every (rows, context) bucket; generation afterwards captures none and gives the plain
    implementation's tokens."""
    folder = H.model_folder("B", "float32", True)
    cfg, w = H.oracle(folder)
    prompts = [H.random_tokens(cfg["vocab_size"], n, seed=n) for n in (2, 7, 20, 3, 11)]
    want = [P.greedy_generate(cfg, w, p, 12) for p in prompts]
    eng = engine_for(folder, use_graphs=True, max_active_requests=5, max_tokens=2048)
    made = eng.warm_up()
    assert made == len(eng.runner.graphs) and made >= 4 and eng.warm_up() == 0
    assert {k[0] for k in eng.runner.graphs} == {1, 2, 4, 8}
    outs = eng.generate(prompts, params(max_tokens=12, temperature=0.0))
    assert [o.token_ids for o in outs] == want
    assert len(eng.runner.graphs) == made and eng.runner.graph_replays > 0
    assert engine_for(folder, use_graphs=False).warm_up() == 0


def test_steps_queued_ahead_give_the_same_tokens_when_requests_stop_arrive_and_are_aborted():
    """With graphs on, the engine queues the next decode step on the GPU, fed with the sampled tokens there, before
    the host has seen the current step's tokens.  A request that stops or is aborted leaves a row in the queued step
    that counts for nothing, one that arrives waits for the queued step; the tokens are those of the plain
    implementation all the same."""
    folder = H.model_folder("A", "float32", True)
    cfg, w = H.oracle(folder)
    prompts = [H.random_tokens(256, n, seed=40 + n) for n in (5, 9, 3, 12)]
    full = [P.greedy_generate(cfg, w, p, 24) for p in prompts]
    eng = engine_for(folder, use_graphs=True)
    # request 0 stops at the token it would produce 10th, request 1 runs to its length
    stop = full[0][9]
    cut0 = full[0][: full[0].index(stop) + 1]
    r0 = eng.add_request(prompts[0], params(max_tokens=24, temperature=0.0, stop_token_ids=[stop]))
    r1 = eng.add_request(prompts[1], params(max_tokens=24, temperature=0.0))
    got = {r0: [], r1: []}
    queued_ahead = 0
    steps = 0
    r2 = r3 = None
    while eng.has_unfinished():
        queued_ahead += eng._ahead is not None
        for ev in eng.step():
            got.setdefault(ev.request_id, []).append(ev.token_id)
        steps += 1
        if steps == 6:                                   # arrives while a queued step exists
            assert eng._ahead is not None
            r2 = eng.add_request(prompts[2], params(max_tokens=24, temperature=0.0))
            got[r2] = []
        if steps == 12:
            r3 = eng.add_request(prompts[3], params(max_tokens=24, temperature=0.0))
            got[r3] = []
        if steps == 16:
            eng.abort(r3)                                # leaves mid-way
    assert queued_ahead > 10
    assert got[r0] == cut0 and got[r1] == full[1] and got[r2] == full[2]
    assert got[r3] == full[3][: len(got[r3])] and 0 < len(got[r3]) < 24
    assert eng.runner.cache.free_pages(0) == eng.runner.cache.paged_groups[0].pool.num_pages
    eng.runner.cache.check()


def test_a_cache_larger_than_device_memory_is_refused_with_its_size():
    from allpaca_amd.cache import CacheTooLarge
    from allpaca_amd.engine import Engine
    folder = H.model_folder("A", "float32", True)
    with pytest.raises(CacheTooLarge, match="GiB"):
        Engine(folder, dtype="float32", page_tokens=16, max_tokens=1 << 34)


@pytest.mark.parametrize("graphs", [False, True])
def test_the_logits_behind_the_tokens_can_be_tapped_and_dumped(tmp_path, graphs):
    """`tap_logits` keeps the logits every token was chosen from (the reference's tap,
    crates/allpaca-core/src/engine.rs:1179-1189); `ALLPACA_LOGITS_DUMP` / `--dump-logits` appends them to a file
    (crates/allpaca-core/src/sampling.rs:100-127).  Greedy tokens are the first maxima of their tapped rows, the rows
    are the plain implementation's logits, and steps queued ahead are tapped like the others."""
    folder = H.model_folder("B", "float32", True)
    cfg, w = H.oracle(folder)
    prompts = [H.random_tokens(1000, n, seed=n) for n in (5, 19)]
    eng = engine_for(folder, use_graphs=graphs)
    eng._dump_path = str(tmp_path / "logits.f32")
    eng.tap_logits(True)
    outs = eng.generate(prompts, params(max_tokens=7, temperature=0.0))
    tapped = eng.take_tapped_logits()
    assert len(tapped) == 14 and eng.take_tapped_logits() == []
    by_request = {}
    for rid, index, row in tapped:
        by_request.setdefault(rid, []).append((index, row))
    for (rid, rows), p, o in zip(sorted(by_request.items()), prompts, outs):
        assert [i for i, _ in rows] == list(range(7))
        assert [int(np.argmax(r)) for _, r in rows] == o.token_ids
        want = P.llama_forward(cfg, w, p + o.token_ids[:-1])[len(p) - 1:]
        assert np.abs(np.stack([r for _, r in rows]) - want).max() < H.F32_ATOL
    dumped = np.fromfile(tmp_path / "logits.f32", dtype="<f4").reshape(-1, 1000)
    assert dumped.shape[0] == 14 and np.array_equal(dumped, np.stack([r for _, _, r in tapped]))
    eng.tap_logits(False)
    eng._dump_path = None
    eng.generate(prompts[:1], params(max_tokens=2, temperature=0.0))
    assert eng.take_tapped_logits() == []
    st = eng.stats
    assert st["prefill_portions"] == 3 and st["batched_rows"] == st["prefill_tokens"] + st["decode_tokens"]
    assert st["pages_in_use"] == 0 and st["pages_in_use_peak"] >= 2 and (st["graph_replays"] > 0) == graphs


def test_a_seed_gives_the_same_weights_on_the_gpu_as_on_the_cpu():
    from allpaca_amd.parts import ParamSpec
    from allpaca_amd.weights import random_tensors
    specs = {"w": ParamSpec((1000, 333)), "n": ParamSpec((77,), store="float32")}
    for dtype in (torch.float32, torch.bfloat16):
        cpu = random_tensors(specs, 5, dtype, norm_std=0.1)
        gpu = random_tensors(specs, 5, dtype, norm_std=0.1, device="cuda:0")
        assert all(torch.equal(cpu[k], gpu[k].cpu()) for k in specs)
