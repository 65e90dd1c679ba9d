#!/usr/bin/env python3
"""Decode and prefill throughput of the engine on Llama-3.1-8B shapes with random weights.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--context 2048] [--layers L]

A step is one decode step of the whole engine (schedule, batch upload, model, sampling, token ids back).
The engine is set up for sequences of up to 8,192 tokens (--max-context), page size 16; the timed decode steps
run with every sequence at 2,048 tokens (--context).
Prints one JSON line: `value` = decoded tokens per second at the given batch; `prefill` = a 2,048-token
prompt in one step; `roofline` = bytes a decode step has to read (every weight once, and the cache of the
live requests) over its time, against 8 TB/s, and beside it what a plain streaming read reaches on this card
(`measured_peak`); `points` = decode at batch 1 and 64.  The way of reporting
follows the reference's bench tool (bytes per token, effective GB/s, share of the peak:
tools/bench/src/roofline.rs:35-70).  Peaks: MI355X HBM3E 8 TB/s; dense bf16 MFMA 2.5 PFLOP/s."""
import argparse
import gc
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}


def build_engine(cfg_json, dtype, batch, context, extra_tokens, layers, seed=0, use_graphs=True, max_context=0,
                 chunk_tokens=2048, pool_tokens=0):
    """An engine on random weights made directly on the GPU (no model folder is written for 16 GB)."""
    import torch

    from allpaca_amd.config import EngineConfig
    from allpaca_amd.engine.engine import Engine
    from allpaca_amd.models import DecoderModel, describe_model
    from allpaca_amd.parts import Runtime
    from allpaca_amd.weights import random_tensors

    cfg_json = dict(cfg_json, num_hidden_layers=layers)
    _, cfg, spec = describe_model(cfg_json)
    model = DecoderModel(spec)
    tdt = torch.bfloat16 if dtype == "bf16" else torch.float32
    page = 16
    # every sequence may grow to `max_context` tokens (positions, block table, pages of the pool)
    per_seq = -(-max(context + extra_tokens, max_context) // page) * page
    ec = EngineConfig(dtype="bfloat16" if dtype == "bf16" else "float32", page_tokens=page,
                      num_pages=(pool_tokens or batch * per_seq) // page + 8, max_active_requests=max(batch, 1),
                      max_batch_tokens=2048, chunk_tokens=chunk_tokens, use_graphs=use_graphs)
    rt = Runtime(torch.device("cuda:0"), tdt, per_seq)
    # weights tensor by tensor on the GPU: nothing of 16 GB passes through host memory
    specs = model.param_specs()
    tensors = {}
    for name, ps in specs.items():
        tensors.update(random_tensors({name: ps}, seed, tdt, 0.02, 0.0, device="cuda:0"))
    model.bind(tensors, rt)
    del tensors
    eng = Engine.from_model(cfg, model, ec)
    return cfg, eng


def weight_bytes(eng):
    """Bytes of every matrix and vector a decode step reads once (the embedding table is read row-wise, a few
    KB, and only counts if the head shares it)."""
    import torch

    from allpaca_amd.kernels.packing import PackedWeight
    seen, total = set(), 0

    def add(v):
        nonlocal total
        if isinstance(v, PackedWeight):
            v = v.data
        if isinstance(v, (tuple, list)):
            for x in v:
                add(x)
        elif isinstance(v, torch.Tensor) and v.dim() >= 1 and v.data_ptr() not in seen:
            seen.add(v.data_ptr())
            total += v.numel() * v.element_size()

    model = eng.model
    add(model.head.weight)
    add(model.final_norm.weight)
    for b in model.blocks:
        for part in b.parts.values():
            for v in vars(part).values():
                add(v)
    return total


def kv_bytes_per_token(eng):
    """Bytes of cache that one more token of a request takes over all layers: what the engine's own estimate of its
    cache says (`CacheEstimate`, from the needs that the model's parts state), a page's bytes over its positions."""
    import torch
    from allpaca_amd.cache import CacheEstimate
    page = eng.config.page_tokens
    elem = torch.empty((), dtype=eng.runner.storage.paged[0].dtype).element_size()
    est = CacheEstimate.of(eng.model.cache_needs(), page, elem)
    return est.bytes_per_page_of_every_group / page


def decode_during_prefill(batch, context, chunk=2048):
    """Tokens the first request may decode while the other prompts are still running in portions of `chunk`."""
    return batch * -(-context // chunk) + batch


def decode_run(eng, cfg, batch, context, steps, warmup, sampled=False):
    """Fills `batch` requests to `context` tokens, then times `steps` decode steps (greedy, or with `sampled` the
    request options' defaults: temperature 0.8, top-k 40, top-p 0.95)."""
    import numpy as np
    import torch

    from allpaca_amd.sampling import GenerationParams
    rng = np.random.default_rng(0)
    # requests that finish their prompt first decode while the others still prefill: leave room for that
    gp = GenerationParams(max_tokens=warmup + steps + decode_during_prefill(batch, context) + 8,
                          **({} if sampled else {"temperature": 0.0}))
    for _ in range(batch):
        eng.add_request(rng.integers(0, cfg.vocab_size, size=context - 1).tolist(), gp)
    while any(not r.decoding for r in eng.scheduler.running) or eng.scheduler.waiting:
        eng.step()
    for _ in range(warmup):
        eng.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    n = 0
    produced = {}
    for _ in range(steps):
        events = eng.step()
        n += len(events)
        for ev in events:
            produced.setdefault(ev.request_id, []).append(ev.token_id)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    assert n == batch * steps, f"{n} tokens from {steps} steps of batch {batch}"
    for rid in list(eng.requests):
        eng.abort(rid)
    decode_run.ids_hash = ids_hash([produced[k] for k in sorted(produced)])   # of the timed steps' tokens
    return dt / steps


def prefill_run(eng, cfg, tokens, repeats=3):
    """One prompt of `tokens` tokens in one step (logits of its last row), best of `repeats`."""
    import numpy as np
    import torch

    from allpaca_amd.engine.batch import Entry
    rng = np.random.default_rng(1)
    best = None
    for i in range(repeats + 1):
        toks = rng.integers(0, cfg.vocab_size, size=tokens).tolist()
        eng.runner.admit(("prefill", i))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        eng.runner.step([Entry(("prefill", i), toks, [tokens - 1])])
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        eng.runner.release(("prefill", i))
        if i > 0:
            best = dt if best is None else min(best, dt)
    return best


def long_prefill_run(eng, cfg, tokens, portion, repeats=2):
    """One prompt of `tokens` tokens in steps of `portion` tokens (logits of its last row only), best of `repeats`.
    Returns the seconds of the whole prompt and of its last step."""
    import numpy as np
    import torch

    from allpaca_amd.engine.batch import Entry
    rng = np.random.default_rng(1)
    best = None
    for i in range(repeats + 1):
        toks = rng.integers(0, cfg.vocab_size, size=tokens).tolist()
        eng.runner.admit(("prompt", i))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for a in range(0, tokens, portion):
            part = toks[a:a + portion]
            if a + portion >= tokens:
                torch.cuda.synchronize()
                t_last = time.perf_counter()
            eng.runner.step([Entry(("prompt", i), part, [len(part) - 1] if a + portion >= tokens else [])])
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        eng.runner.release(("prompt", i))
        if i > 0 and (best is None or t1 - t0 < best[0]):
            best = (t1 - t0, t1 - t_last)
    return best


def ids_hash(token_lists):
    """A short hash of produced token ids (requests in order): the same run gives the same hash."""
    import hashlib
    h = hashlib.sha256()
    for toks in token_lists:
        h.update((",".join(str(int(t)) for t in toks) + ";").encode())
    return h.hexdigest()[:16]


def requests_run(eng, cfg, n_requests, min_prompt, max_prompt, new_tokens, seed=0, sampled=False):
    """`n_requests` requests with prompts of random length arrive at once and run to `new_tokens` tokens each
    through the scheduler: portions of prompts beside decoding rows.  Returns a dict of totals and mean times."""
    import numpy as np
    import torch

    from allpaca_amd.sampling import GenerationParams
    rng = np.random.default_rng(seed)
    lengths = [int(x) for x in rng.integers(min_prompt, max_prompt + 1, size=n_requests)]
    # greedy, or the defaults of the request options (temperature 0.8, top-k 40, top-p 0.95)
    gp = GenerationParams(max_tokens=new_tokens) if sampled else GenerationParams(max_tokens=new_tokens, temperature=0.0)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ids = [eng.add_request(rng.integers(0, cfg.vocab_size, size=n).tolist(), gp) for n in lengths]
    reqs = [eng.requests[i] for i in ids]
    steps = 0
    while eng.has_unfinished():
        eng.step()
        steps += 1
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    times = [r.timing() for r in reqs]
    out_tokens = sum(len(r.output) for r in reqs)
    assert out_tokens == n_requests * new_tokens, f"{out_tokens} tokens from {n_requests} requests"
    ttft = [1e3 * t["ttft"] for t in times]
    itl = [1e3 * t["itl"] for t in times]
    return {"seconds": dt, "steps": steps, "prompt_tokens": sum(lengths), "output_tokens": out_tokens,
            "ttft_ms": float(np.mean(ttft)), "itl_ms": float(np.mean(itl)),
            "ttft_p50_ms": float(np.percentile(ttft, 50)), "ttft_p95_ms": float(np.percentile(ttft, 95)),
            "itl_p50_ms": float(np.percentile(itl, 50)), "itl_p95_ms": float(np.percentile(itl, 95)),
            "ids_hash": ids_hash([r.output for r in reqs]),
            "preemptions": eng.scheduler.preemption_count}


def prefill_flops(cfg, layers, T):
    D, F, V = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    H, Hk, d = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
    linear = 2 * T * D * ((H + 2 * Hk) * d + H * d) + 2 * T * D * 3 * F
    attn = 2 * 2 * H * d * (T * (T + 1) // 2)
    return layers * (linear + attn) + 2 * D * V


# ---- per-kernel times (a pass of its own, never inside the measured steps) -----------------------------------
# entry point -> (indices of M, N, K among its int arguments, matrices read); N of the q/k/v product comes from its heads
_PRODUCTS = {
    "apc_skinny_gemm_bf16": ((2, 3, 4), 1), "apc_skinny_gemm_emit_bf16": ((2, 3, 4), 1),
    "apc_skinny_gemm_pre_bf16": ((3, 4, 5), 1), "apc_skinny_swiglu_bf16": ((2, 3, 4), 2),
    "apc_skinny_swiglu_pre_bf16": ((3, 4, 5), 2), "apc_gemm_bf16": ((2, 3, 4), 1), "apc_gemm_swiglu_bf16": ((2, 3, 4), 2),
    "apc_gemm_splitk_emit_bf16": ((2, 3, 4), 1), "apc_gemm_direct_emit_bf16": ((2, 3, 4), 1),
}


def _product_work(name, ints):
    """(rows, weight bytes read, flops) of one call of a matrix product's entry point, or None."""
    if name in _PRODUCTS:
        (m, n, k), mats = _PRODUCTS[name]
        M, N, K = ints[m], ints[n], ints[k]
    elif name in ("apc_skinny_qkv_rope_bf16", "apc_gemm_splitk_qkv_rope_bf16"):
        M, K, H, Hk, d = ints[3:8]
        N, mats = (H + 2 * Hk) * d, 1
    elif name in ("apc_gemm_pre_bf16", "apc_gemm_splitk_pre_bf16"):
        M, N, K, mode = ints[3:7]
        mats = 2 if mode == 3 else 1
    elif name == "apc_gemm_splitk_bf16":
        M, N, K, mode = ints[2:6]
        mats = 2 if mode == 3 else 1
    else:
        return None
    return M, mats * N * K * 2, 2 * mats * M * N * K


def kernel_table(totals, steps, attention_bytes=0, attention_flops=0):
    """Per entry point: calls and microseconds a step, and for the products and the attention what they read or
    compute and at what rate, against the published peaks."""
    rows = []
    for name, t in sorted(totals.items(), key=lambda kv: -kv[1]["us"]):
        r = {"kernel": name, "calls": round(t["calls"] / steps, 1), "us": round(t["us"] / steps, 1)}
        works = [_product_work(name, a) for a in t["args"]]
        nbytes = flops = 0
        if works and works[0] is not None:
            nbytes, flops = sum(w[1] for w in works) / steps, sum(w[2] for w in works) / steps
            r["rows"] = works[0][0]
        elif name == "apc_attention_decode_bf16":
            nbytes = attention_bytes
        elif name == "apc_attention_prefill_bf16":
            flops = attention_flops
        sec = t["us"] / steps * 1e-6
        if nbytes and (not flops or flops / nbytes < 300):     # below the ridge: bound by reading
            r.update({"GB": round(nbytes / 1e9, 3), "GB/s": round(nbytes / sec / 1e9, 1),
                      "frac_hbm": round(nbytes / sec / 1e9 / HBM_PEAK_GBS, 3)})
        elif flops:
            r.update({"TFLOP": round(flops / 1e12, 3), "TFLOP/s": round(flops / sec / 1e12, 1),
                      "frac_mfma": round(flops / sec / PEAK_FLOPS["bf16"], 3)})
        rows.append(r)
    return rows


def kernel_times(cfg_json, args, layers):
    """Event timers around every kernel launch of a decode step, a 2,048-token prefill and a mixed step (a portion of
    512 tokens beside the decoding rows), run eagerly in passes of their own; and the host's time to launch a mixed step."""
    import numpy as np
    import torch

    from allpaca_amd.engine.batch import Entry
    from allpaca_amd.kernels import lib as klib
    from allpaca_amd.sampling import GenerationParams
    B, ctx = args.batch, args.context
    cfg, eng = build_engine(cfg_json, args.dtype, B + 1, ctx, 600, layers, use_graphs=False, max_context=args.max_context)
    rng = np.random.default_rng(0)
    gp = GenerationParams(max_tokens=64, temperature=0.0)
    for _ in range(B):
        eng.add_request(rng.integers(0, cfg.vocab_size, size=ctx - 1).tolist(), gp)
    while any(not r.decoding for r in eng.scheduler.running) or eng.scheduler.waiting:
        eng.step()
    for _ in range(3):
        eng.step()
    out = {}
    steps = 4
    # The tables come from timers around the entry points as Python calls them, so these passes walk the model's
    # parts in Python (the same kernels with the same arguments as the compiled executor issues); the host's time to
    # launch a step is measured on both.
    native, eng.runner.native = eng.runner.native, None
    with klib.timing() as t:
        for _ in range(steps):
            eng.step()
    kv = kv_bytes_per_token(eng)
    out[f"decode_b{B}_ctx{ctx}"] = kernel_table(t.totals(), steps, attention_bytes=B * (ctx + 5) * kv)
    # a mixed step: a portion of a new prompt beside the B decoding rows, as long as the scheduler makes it (a chunk of
    # 512 tokens, cut back so that the step's rows are whole tiles); host time = until the launches are queued
    ids = [r.id for r in eng.scheduler.running]
    eng.runner.admit("mixed")
    tile = eng.scheduler.row_tile
    portion = 512
    if tile and 0 < (portion + B) % tile <= tile // 4:
        portion -= (portion + B) % tile
    mixed = lambda at: [Entry("mixed", rng.integers(0, cfg.vocab_size, size=portion).tolist(), [portion - 1])] + \
        [Entry(i, [1], [0]) for i in ids]
    def launch_time(reps=3):
        eng.runner.step(mixed(0))
        torch.cuda.synchronize()
        host, gpu = [], []
        for rep in range(reps):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            batch = mixed(rep)
            t0 = time.perf_counter()
            e0.record()
            eng.runner.step(batch)
            e1.record()
            host.append((time.perf_counter() - t0) * 1e6)
            e1.synchronize()
            gpu.append(e0.elapsed_time(e1) * 1e3)
        return round(min(host), 1), round(min(gpu), 1)

    walk_host, walk_gpu = launch_time()
    with klib.timing() as t:
        eng.runner.step(mixed(9))
    hd = cfg.num_attention_heads * cfg.head_dim
    out[f"mixed_{portion}_plus_b{B}"] = kernel_table(t.totals(), 1, attention_bytes=B * ctx * kv,
                                                     attention_flops=layers * 4 * hd * portion * (portion * 4 + portion // 2))
    eng.runner.native = native
    host, gpu = launch_time() if native is not None else (walk_host, walk_gpu)
    out["host_us_mixed_step"] = {"host_launch_us": host, "gpu_us": gpu, "executor": "compiled" if native is not None else "python",
                                 "python_walk_host_launch_us": walk_host, "python_walk_gpu_us": walk_gpu}
    eng.runner.native = None
    eng.runner.release("mixed")
    # prefill of 2,048 tokens in one step
    T = 2048
    eng.runner.admit("pf")
    eng.runner.step([Entry("pf", rng.integers(0, cfg.vocab_size, size=T).tolist(), [T - 1])])
    eng.runner.release("pf")
    eng.runner.admit("pf2")
    with klib.timing() as t:
        eng.runner.step([Entry("pf2", rng.integers(0, cfg.vocab_size, size=T).tolist(), [T - 1])])
    out[f"prefill_{T}"] = kernel_table(t.totals(), 1, attention_flops=layers * 4 * hd * (T * (T + 1) // 2))
    eng.runner.native = native
    return out


def sampler_times(vocab: int) -> dict:
    """Microseconds to choose the tokens of 1, 8 and 64 rows of random logits under four rules.  `gpu_us`: the
    kernels alone, their launches queued while the GPU is busy with something else (as a serving loop queues them
    behind the step), so that no waiting for the host is in it; `latency_us`: `Sampler.sample` from call to token ids
    on an idle GPU (parameters up, kernels, ids back)."""
    import torch
    from allpaca_amd.kernels import ops
    from allpaca_amd.sampling import GenerationParams
    from allpaca_amd.sampling.sampler import Sampler
    dev = torch.device("cuda:0")
    rules = {"greedy": dict(temperature=0.0, top_k=0, top_p=1.0),
             "temperature": dict(temperature=0.8, top_k=0, top_p=1.0),
             "top_k_40_top_p_0.95": dict(temperature=0.8, top_k=40, top_p=0.95),
             "top_p_0.95": dict(temperature=0.8, top_k=0, top_p=0.95)}
    busy = torch.randn(8192, 8192, device=dev)
    sampler = Sampler(dev, 0)
    out = {}
    for rows in (1, 8, 64):
        logits = torch.randn(rows, vocab, device=dev) * 3.0
        ids = torch.empty(rows, dtype=torch.int32, device=dev)
        u = torch.rand(rows, device=dev)
        for name, rule in rules.items():
            params = [GenerationParams(max_tokens=1, **rule) for _ in range(rows)]
            t = torch.full((rows,), rule["temperature"], device=dev)
            k = torch.full((rows,), rule["top_k"], dtype=torch.int32, device=dev)
            p = torch.full((rows,), rule["top_p"], device=dev)

            def kernels():
                if name == "greedy":
                    ops.argmax_rows(logits, ids)
                else:
                    ops.sample_rows(logits, t, k, p, u, ids, any_top_k=rule["top_k"] > 0, any_top_p=rule["top_p"] < 1.0,
                                    few_after_top_k=0 < rule["top_k"] <= 1024)
            calls = 20
            for _ in range(3):
                kernels()
                sampler.sample(logits, params, [0] * rows)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            for _ in range(6):
                busy @ busy                                   # a few milliseconds for the launches to queue behind
            e0.record()
            for _ in range(calls):
                kernels()
            e1.record()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for i in range(calls):
                sampler.sample(logits, params, [i] * rows)
            wall = time.perf_counter() - t0
            out[f"b{rows}_{name}"] = {"gpu_us": round(e0.elapsed_time(e1) * 1e3 / calls, 1),
                                      "latency_us": round(wall * 1e6 / calls, 1)}
    return out


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=2048, help="tokens every sequence holds when the decode steps are timed")
    ap.add_argument("--max-context", type=int, default=8192,
                    help="tokens a sequence may grow to: positions, block tables and the page pool are made for it")
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the configuration (0: all)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--preset", default="llama-3.1-8b")
    ap.add_argument("--no-points", action="store_true", help="skip the batch-1 and batch-64 points and the prefill")
    ap.add_argument("--no-graphs", action="store_true")
    ap.add_argument("--requests", type=int, default=0,
                    help="instead of the decode steps: this many requests with prompts of --min-prompt..--max-prompt "
                         "tokens arrive at once and decode --new-tokens tokens each under chunked prefill")
    ap.add_argument("--min-prompt", type=int, default=128)
    ap.add_argument("--max-prompt", type=int, default=4096)
    ap.add_argument("--new-tokens", type=int, default=256)
    ap.add_argument("--chunk", type=int, default=512, help="largest portion of a prompt in a step (with --requests)")
    ap.add_argument("--sampled", action="store_true",
                    help="tokens drawn with temperature 0.8, top-k 40, top-p 0.95 instead of greedy (the decode steps, or "
                         "with --requests the requests)")
    ap.add_argument("--kernel-times", action="store_true",
                    help="instead of the measured steps: event timers around every kernel of a decode step, a mixed step "
                         "and a 2,048-token prefill (eager passes of their own), and the host's time to launch a mixed step")
    ap.add_argument("--prompt", type=int, default=0,
                    help="with --only prefill: a prompt of this many tokens in steps of --portion tokens instead of the "
                         "2,048-token prompt in one step")
    ap.add_argument("--portion", type=int, default=2048)
    ap.add_argument("--only", choices=["decode", "prefill", "sampler"], default=None,
                    help="for profiling: only the decode steps at --batch (as --no-points), only the 2,048-token "
                         "prefill (prints its figures as the line's value), or only the sampler over the preset's "
                         "vocabulary (microseconds a step's rows take on the GPU and on the host)")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported", flush=True)
        return 2

    import torch

    from allpaca_amd.config import preset
    from allpaca_amd.kernels import lib as klib
    cfg_json = preset(args.preset)
    full_layers = cfg_json["num_hidden_layers"]
    layers = args.layers or full_layers
    klib.load("plain")
    klib.load("tuned")

    if args.kernel_times:
        print(json.dumps({"metric": "microseconds per kernel and step (event timers, eager passes)", "unit": "us",
                          "n_gpus": 1, "dtype": args.dtype,
                          "config": {"model": args.preset, "layers": layers, "layers_of_configuration": full_layers,
                                     "global_batch": args.batch, "seq_len": args.context},
                          "kernel_times": kernel_times(cfg_json, args, layers)}), flush=True)
        return 0
    if args.requests:
        n = args.requests
        top = args.max_prompt + args.new_tokens
        cfg, eng = build_engine(cfg_json, args.dtype, n, top, 0, layers, use_graphs=not args.no_graphs,
                                max_context=top, chunk_tokens=args.chunk, pool_tokens=n * (top + 16))
        t0 = time.perf_counter()
        captured = eng.warm_up()                                                                    # decode graphs
        requests_run(eng, cfg, min(n, 4), args.min_prompt, min(args.max_prompt, 512), 8, seed=1)   # first launches
        warm = time.perf_counter() - t0
        r = requests_run(eng, cfg, n, args.min_prompt, args.max_prompt, args.new_tokens, sampled=args.sampled)
        print(json.dumps({
            "metric": f"output tok/s, {n} requests at once, prompts {args.min_prompt}-{args.max_prompt}, "
                      f"{args.new_tokens} new tokens each, chunked prefill"
                      + (", sampled (temperature 0.8, top-k 40, top-p 0.95)" if args.sampled else ""),
            "value": round(r["output_tokens"] / r["seconds"], 1), "unit": "tok/s", "n_gpus": 1,
            "seconds": round(r["seconds"], 3), "steps": r["steps"], "prompt_tokens": r["prompt_tokens"],
            "output_tokens": r["output_tokens"], "all_tokens_per_s": round((r["prompt_tokens"] + r["output_tokens"]) / r["seconds"], 1),
            "mean_ttft_ms": round(r["ttft_ms"], 1), "mean_itl_ms": round(r["itl_ms"], 2),
            "ttft_p50_ms": round(r["ttft_p50_ms"], 1), "ttft_p95_ms": round(r["ttft_p95_ms"], 1),
            "itl_p50_ms": round(r["itl_p50_ms"], 2), "itl_p95_ms": round(r["itl_p95_ms"], 2),
            "ids_hash": r["ids_hash"], "preemptions": r["preemptions"],
            "graphs_captured_before": captured, "warm_up_seconds": round(warm, 2),
            "dtype": args.dtype, "data": "synthetic: random N(0, 0.02) weights, uniform random token ids",
            "config": {"model": args.preset, "layers": layers, "layers_of_configuration": full_layers,
                       "chunk_tokens": args.chunk, "max_batch_tokens": 2048, "page_tokens": 16}}), flush=True)
        return 0
    if args.only == "sampler":
        print(json.dumps({"metric": "microseconds to choose a step's tokens (GPU time, launches queued behind other work)",
                          "unit": "us", "n_gpus": 1, "config": {"model": args.preset, "vocab": cfg_json["vocab_size"]},
                          "sampler": sampler_times(cfg_json["vocab_size"])}), flush=True)
        return 0
    if args.only == "decode":
        args.no_points = True
    if args.only == "prefill" and args.prompt > 0:
        T = args.prompt
        cfg, eng = build_engine(cfg_json, args.dtype, 1, T, 64, layers, use_graphs=not args.no_graphs,
                                max_context=max(args.max_context, T + 64))
        psec, last = long_prefill_run(eng, cfg, T, args.portion)
        fl = prefill_flops(cfg, layers, T)
        print(json.dumps({"metric": f"prefill tok/s, one prompt of {T} tokens in steps of {args.portion}",
                          "value": round(T / psec, 1), "unit": "tok/s", "n_gpus": 1, "seconds": round(psec, 4),
                          "last_step_ms": round(last * 1e3, 3), "dtype": args.dtype,
                          "frac_of_mfma_peak": round(fl / psec / PEAK_FLOPS[args.dtype], 4),
                          "config": {"model": args.preset, "layers": layers, "prompt_tokens": T,
                                     "portion": args.portion}}), flush=True)
        return 0
    if args.only == "prefill":
        T = 2048
        cfg, eng = build_engine(cfg_json, args.dtype, 1, T, 64, layers, use_graphs=not args.no_graphs,
                                max_context=args.max_context)
        psec = prefill_run(eng, cfg, T)
        fl = prefill_flops(cfg, layers, T)
        print(json.dumps({"metric": "prefill tok/s @ 2048 tokens", "value": round(T / psec, 1), "unit": "tok/s",
                          "n_gpus": 1, "ms_per_step": round(psec * 1e3, 3), "dtype": args.dtype,
                          "frac_of_mfma_peak": round(fl / psec / PEAK_FLOPS[args.dtype], 4),
                          "config": {"model": args.preset, "layers": layers}}), flush=True)
        return 0

    # what this card delivers: a streaming read of 8 GiB and a loop of MFMAs from registers (allpaca_amd/csrc/probe.hip)
    from allpaca_amd.kernels import probe
    measured_gbs = probe.read_bandwidth(8.0)
    measured_tflops = probe.mfma_rate() if args.dtype == "bf16" else None
    points = {}
    batches = [args.batch] + ([] if args.no_points else [b for b in (1, 64) if b != args.batch])
    ms = {}
    prefill = None
    roof = None
    for b in batches:
        extra = args.warmup + args.steps + decode_during_prefill(b, args.context) + 16
        cfg, eng = build_engine(cfg_json, args.dtype, max(b, 1), args.context, extra, layers,
                                use_graphs=not args.no_graphs, max_context=args.max_context)
        sec = decode_run(eng, cfg, b, args.context, args.steps, args.warmup, sampled=args.sampled)
        ms[b] = sec * 1e3
        if b == args.batch:
            main_hash = decode_run.ids_hash
            wbytes = weight_bytes(eng)
            ctx_mid = args.context + args.warmup + args.steps // 2
            total = wbytes + b * ctx_mid * kv_bytes_per_token(eng)
            gbs = total / sec / 1e9
            roof = {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                    "frac": round(gbs / HBM_PEAK_GBS, 4), "measured_peak": round(measured_gbs, 1),
                    "frac_of_measured": round(gbs / measured_gbs, 4)}
            if not args.no_points:
                T = 2048
                psec = prefill_run(eng, cfg, T)
                fl = prefill_flops(cfg, layers, T)
                prefill = {"value": round(T / psec, 1), "tokens": T, "ms": round(psec * 1e3, 3),
                           "frac": round(fl / psec / PEAK_FLOPS[args.dtype], 4)}
                if measured_tflops:
                    prefill["measured_peak_tflops"] = round(measured_tflops, 1)
        else:
            points[f"decode_b{b}"] = round(b / sec, 1)
        del eng
        gc.collect()                 # an engine holds cycles (graphs, parts): without this the next one is built beside it
        torch.cuda.empty_cache()

    sec = ms[args.batch] / 1e3
    out = {
        "metric": f"decode tok/s @ batch {args.batch}, context {args.context} ({args.preset} shapes)"
                  + (", sampled (temperature 0.8, top-k 40, top-p 0.95)" if args.sampled else ""),
        "value": round(args.batch / sec, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms[args.batch], 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic: random N(0, 0.02) weights, uniform random token ids",
        "config": {
            "model": args.preset, "layers": layers, "layers_of_configuration": full_layers,
            "hidden_size": cfg.hidden_size, "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim, "intermediate_size": cfg.intermediate_size, "vocab_size": cfg.vocab_size,
            "rope_theta": cfg.rope_theta, "rope_scaling_factor": cfg.rope_scaling.factor if cfg.rope_scaling else 1.0,
            "rms_norm_eps": cfg.rms_norm_eps, "tied_head": cfg.tie_word_embeddings, "global_batch": args.batch,
            "seq_len": args.context, "max_context": max(args.max_context, args.context), "page_tokens": 16,
            "parallelism": "single GPU",
            "graphs": not args.no_graphs,
        },
    }
    out["ids_hash"] = main_hash      # of the tokens the timed steps produced (greedy): the same run, the same hash
    if prefill:
        out["prefill"] = prefill
    if roof:
        out["roofline"] = roof
    if points:
        out["points"] = points
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
