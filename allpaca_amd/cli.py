"""Command line.  Options carry the reference's names where it has them
(`allpaca-server`: --config, --model, --synthetic, --seed, --cpu-only,
crates/allpaca-server/src/cli.rs:11-72; the TOML sections [engine], [prefill],
[kv], [sampling] of allpaca.example.toml) and settings are merged in its order:
compiled defaults, then the TOML file, then flags
(crates/allpaca-types/src/config.rs:56-98).  There is no server here: the
subcommands are `generate` (token ids in, token ids out), `replay` (bin/trace_run)
and `bench`."""
from __future__ import annotations

import argparse
import json
import os
import sys
import time
from typing import List, Optional


def _token_lists(spec: str) -> List[List[int]]:
    """"1,2,3" is one prompt; "1,2;4,5" two; "@file" reads one prompt per line."""
    if spec.startswith("@"):
        with open(spec[1:]) as f:
            lines = [ln.strip() for ln in f if ln.strip()]
    else:
        lines = [p for p in spec.split(";") if p.strip()]
    return [[int(t) for t in ln.replace(",", " ").split()] for ln in lines]


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(prog="allpaca-amd", description="Single-GPU llama inference engine for MI355X")
    sub = ap.add_subparsers(dest="command", required=True)
    g = sub.add_parser("generate", help="generate token ids for prompts given as token ids")
    g.add_argument("--config", help="TOML file; flags override it, it overrides the defaults")
    g.add_argument("--model", help="folder with config.json and model.safetensors")
    g.add_argument("--synthetic", nargs="?", const="llama-tiny-a", metavar="PRESET",
                   help="random weights of a preset shape instead of --model (default preset llama-tiny-a)")
    g.add_argument("--seed", type=int, help="seed of the random weights and of sampling")
    g.add_argument("--dtype", choices=["bfloat16", "float32", "bf16", "fp32"])
    g.add_argument("--cpu-only", action="store_true", help="refused: this engine has no CPU path")
    g.add_argument("--prompt-tokens", required=True, help='"1,2,3", several prompts as "1,2;3,4", or @file')
    g.add_argument("--max-tokens", type=int)
    g.add_argument("--temperature", type=float)
    g.add_argument("--top-k", type=int)
    g.add_argument("--top-p", type=float)
    g.add_argument("--stop-token-ids", help="comma-separated ids")
    g.add_argument("--page-tokens", type=int)
    g.add_argument("--num-pages", type=int)
    g.add_argument("--chunk-tokens", type=int)
    g.add_argument("--max-batch-tokens", type=int)
    g.add_argument("--max-active-requests", type=int)
    g.add_argument("--json", action="store_true", help="print one JSON object per prompt")
    g.add_argument("--dump-logits", metavar="FILE",
                   help="append the logits every token is chosen from to FILE, a vocabulary per token as little-endian "
                        "float32 (what ALLPACA_LOGITS_DUMP=FILE does for any program)")
    r = sub.add_parser("replay", help="trace replay (same as bin/trace_run)")
    r.add_argument("rest", nargs=argparse.REMAINDER)
    b = sub.add_parser("bench", help="decode and prefill throughput (same as bench.py)")
    b.add_argument("rest", nargs=argparse.REMAINDER)
    return ap


def _load_toml(path: Optional[str]) -> dict:
    if not path:
        return {}
    import tomli
    with open(path, "rb") as f:
        return tomli.load(f)


def settings_from(args) -> tuple:
    """(EngineConfig, GenerationParams, model folder or None, preset or None)"""
    from .config import EngineConfig
    from .sampling import GenerationParams
    toml = _load_toml(args.config)
    ec, gp = EngineConfig(), GenerationParams()
    t_engine, t_prefill, t_kv = toml.get("engine", {}), toml.get("prefill", {}), toml.get("kv", {})
    t_samp, t_model = toml.get("sampling", {}), toml.get("model", {})
    for key, src in (("max_active_requests", t_engine), ("chunk_tokens", t_prefill), ("page_tokens", t_kv),
                     ("num_pages", t_kv), ("max_batch_tokens", t_engine), ("dtype", t_engine), ("seed", t_engine)):
        if key in src:
            setattr(ec, key, src[key])
    for key in ("temperature", "top_k", "top_p", "max_tokens"):
        if key in t_samp:
            setattr(gp, key, t_samp[key])
    model = t_model.get("path")
    for key in ("page_tokens", "num_pages", "chunk_tokens", "max_batch_tokens", "max_active_requests"):
        v = getattr(args, key)
        if v is not None:
            setattr(ec, key, v)
    if args.dtype:
        ec.dtype = {"bf16": "bfloat16", "fp32": "float32"}.get(args.dtype, args.dtype)
    if args.seed is not None:
        ec.seed = args.seed
        gp.seed = args.seed
    for key in ("max_tokens", "temperature", "top_k", "top_p"):
        v = getattr(args, key)
        if v is not None:
            setattr(gp, key, v)
    if args.stop_token_ids:
        gp.stop_token_ids = [int(t) for t in args.stop_token_ids.split(",") if t.strip()]
    if args.model:
        model = args.model
    return ec, gp, model, args.synthetic


def cmd_generate(args) -> int:
    if args.cpu_only:
        print("allpaca-amd: --cpu-only is not available: every step runs on HIP kernels", file=sys.stderr)
        return 2
    from .config import preset
    from .engine import Engine
    ec, gp, model, synthetic = settings_from(args)
    prompts = _token_lists(args.prompt_tokens)
    longest = max(len(p) for p in prompts) + gp.max_tokens
    if not ec.num_pages:
        ec.max_tokens = max(64, sum(-(-(len(p) + gp.max_tokens) // 64) * 64 for p in prompts))
    if synthetic:
        engine = Engine.synthetic(preset(synthetic), seed=ec.seed, config=ec)
    elif model:
        engine = Engine(model, ec)
    else:
        print("allpaca-amd: give --model DIR or --synthetic [PRESET]", file=sys.stderr)
        return 2
    if args.dump_logits:
        engine._dump_path = args.dump_logits
    t0 = time.time()
    outs = engine.generate(prompts, gp)
    dt = time.time() - t0
    for p, o in zip(prompts, outs):
        if args.json:
            print(json.dumps(dict(prompt_tokens=o.prompt_tokens, completion_tokens=o.completion_tokens,
                                  token_ids=o.token_ids, finish_reason=o.finish_reason,
                                  queue_ms=_ms(o.timing["queue"]), ttft_ms=_ms(o.timing["ttft"]),
                                  itl_ms=_ms(o.timing["itl"]))))
        else:
            print(" ".join(str(t) for t in o.token_ids))
    n = sum(o.completion_tokens for o in outs)
    print(f"{n} tokens in {dt:.3f} s ({n / dt:.1f} tok/s), {engine.stats['steps']} steps, "
          f"{engine.stats['preemptions']} preemptions, {engine.stats['prefill_portions']} prompt portions, "
          f"{engine.stats['graph_replays']} graph replays, at most {engine.stats['pages_in_use_peak']} pages in use",
          file=sys.stderr)
    return 0


def _ms(seconds):
    return None if seconds is None else round(seconds * 1e3, 3)


def main(argv: Optional[List[str]] = None) -> int:
    args = build_parser().parse_args(argv)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    if args.command == "generate":
        return cmd_generate(args)
    import subprocess
    rest = [a for a in args.rest if a != "--"]
    target = [sys.executable, os.path.join(root, "bin", "trace_run")] if args.command == "replay" else \
             [sys.executable, os.path.join(root, "bench.py")]
    return subprocess.call(target + rest)   # a child process, so nothing that touched the GPU is replaced


if __name__ == "__main__":
    sys.exit(main())
