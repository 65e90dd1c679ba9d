"""Random streams of requests through the whole engine: arrivals at different steps, stop ids, aborts, pools so
small that requests are preempted and recomputed, decode steps replayed as graphs and queued ahead of the host,
in 32-bit and in bfloat16, on two tiny configurations.  A fixed list of seeds; every run is bounded.
In spirit: crates/allpaca-core/tests/hip_runtime.rs:8032-8200 (tokens under concurrency equal the solo tokens)."""
import numpy as np
import pytest

import helpers as H
import plain_llama as P

pytestmark = pytest.mark.gpu

SEEDS = [1, 2, 3, 5, 8, 13]
preemptions_seen = {"float32": 0, "bfloat16": 0}


def scenario(name, seed):
    rng = np.random.default_rng(seed)
    V = H.CONFIGS[name][0]["vocab_size"]
    n_req = int(rng.integers(3, 10))
    prompts = [H.random_tokens(V, int(rng.integers(1, 50)), seed=seed * 50 + i) for i in range(n_req)]
    new = [int(rng.integers(1, 20)) for _ in range(n_req)]
    sampled = [bool(rng.random() < 0.25) for _ in range(n_req)]
    page = int(rng.choice([8, 16]))
    biggest = max(len(p) + n for p, n in zip(prompts, new))
    # room for the largest request and at most a few pages more: requests must give way to each other
    pool = -(-biggest // page) * page + int(rng.integers(0, 4)) * page * int(rng.integers(1, 4))
    opts = dict(page_tokens=page, max_tokens=pool, max_active_requests=int(rng.integers(1, 7)),
                chunk_tokens=int(rng.integers(2, 33)), max_batch_tokens=int(rng.integers(4, 65)),
                use_graphs=bool(rng.random() < 0.7))
    arrive = sorted(int(rng.integers(0, 25)) for _ in range(n_req))
    abort_at = {i: int(rng.integers(1, 30)) for i in range(n_req) if rng.random() < 0.15}
    stop_draw = [(float(rng.random()), float(rng.random())) for _ in range(n_req)]
    return prompts, new, sampled, opts, arrive, abort_at, stop_draw


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
@pytest.mark.parametrize("seed", SEEDS)
def test_random_streams_of_requests(name, dtype, seed):
    from allpaca_amd.engine import Engine
    from allpaca_amd.sampling import GenerationParams
    folder = H.model_folder(name, dtype, True)
    cfg, w = H.oracle(folder)
    prompts, new, sampled, opts, arrive, abort_at, stop_draw = scenario(name, seed)
    n_req = len(prompts)
    # the plain implementation's greedy continuation; a stop id is one of its tokens (for some requests)
    full = [P.greedy_generate(cfg, w, p, n) for p, n in zip(prompts, new)]
    stops = [([f[int(b * len(f))]] if a < 0.3 else []) for f, (a, b) in zip(full, stop_draw)]

    def params(i):
        if sampled[i]:
            return GenerationParams(max_tokens=new[i], temperature=0.9, top_k=20, top_p=0.9, seed=1000 + i,
                                    stop_token_ids=stops[i])
        return GenerationParams(max_tokens=new[i], temperature=0.0, stop_token_ids=stops[i])

    eng = Engine(folder, dtype=dtype, **opts)
    ids, got, aborted = {}, {}, set()
    step = nxt = 0
    while nxt < n_req or eng.has_unfinished():
        while nxt < n_req and arrive[nxt] <= step:
            ids[nxt] = eng.add_request(prompts[nxt], params(nxt))
            got[ids[nxt]] = []
            nxt += 1
        for ev in eng.step():
            got[ev.request_id].append(ev.token_id)
        step += 1
        for i, at in abort_at.items():
            if at == step and i in ids and i not in aborted:
                eng.abort(ids[i])
                aborted.add(i)
        eng.runner.cache.check()
        assert step < 400, "the stream of requests does not end"
    preemptions_seen[dtype] += eng.scheduler.preemption_count
    cache = eng.runner.cache
    assert cache.free_pages(0) == cache.paged_groups[0].pool.num_pages and not cache.live()

    solo = None
    for i in range(n_req):
        out = got[ids[i]]
        where = f"{name} {dtype} seed {seed} request {i} ({opts})"
        # how a request ends: at its first stop id, at max_tokens, or where it was aborted
        cut = [j for j, t in enumerate(out) if t in stops[i]]
        assert not cut or cut[0] == len(out) - 1, where
        if i not in aborted:
            assert len(out) == new[i] or (out and out[-1] in stops[i]), where
        if sampled[i]:
            if dtype == "float32":
                # 32-bit rows do not depend on the batch, the cutting or a recomputation: the same tokens as alone
                solo = solo or Engine(folder, dtype=dtype, page_tokens=16, max_tokens=256, use_graphs=False)
                alone = solo.generate([prompts[i]], params(i))[0].token_ids
                assert out == alone[:len(out)], where
            continue
        if dtype == "float32":
            want = full[i][: full[i].index(stops[i][0]) + 1] if stops[i] and stops[i][0] in full[i] else full[i]
            assert out == want[:len(out)], (where, out, want)
        elif out:
            # bfloat16 may leave the plain path at a near tie (and a recomputed request takes other kernels than a
            # decoded one): every token is the plain implementation's choice for its own context, or within
            # bfloat16's noise of it
            lg = H.oracle_logits(folder, prompts[i] + out[:-1])[len(prompts[i]) - 1:]
            for j, t in enumerate(out):
                assert lg[j].max() - lg[j][t] <= 0.02 * np.abs(lg[j]).max(), (where, j, t)


def test_the_streams_made_requests_give_way():
    """The scenarios above are only worth their name if pages ran out in some of them."""
    if not any(preemptions_seen.values()):
        pytest.skip("runs after test_random_streams_of_requests")
    assert preemptions_seen["float32"] > 0 and preemptions_seen["bfloat16"] > 0, preemptions_seen
