"""The programs' contracts that can be checked without a GPU: bench.py refuses more than one GPU with one line and
exit code 2; the command line refuses the CPU; trace_run and the command line show their options."""
import json
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run(*cmd, timeout=120):
    return subprocess.run([sys.executable, *cmd], capture_output=True, text=True, timeout=timeout, cwd=ROOT)


def test_bench_refuses_more_than_one_gpu_with_one_line():
    r = run("bench.py", "--gpus", "2", "--steps", "1", "--warmup", "0")
    assert r.returncode == 2
    lines = [ln for ln in r.stdout.strip().splitlines() if ln.strip()]
    assert len(lines) == 1 and "one GPU" in lines[0]


def test_bench_defaults_are_the_named_configuration():
    sys.path.insert(0, ROOT)
    from allpaca_amd.config import preset
    cfg = preset("llama-3.1-8b")
    base = json.load(open(os.path.join(ROOT, "BASELINE.json")))
    text = base["configs"][2]
    for key, word in (("num_hidden_layers", "32 layers"), ("hidden_size", "hidden 4096"), ("num_attention_heads", "32 heads"),
                      ("num_key_value_heads", "8 KV heads"), ("intermediate_size", "intermediate 14336"),
                      ("vocab_size", "vocab 128256")):
        assert word.split()[0 if word[0].isdigit() else 1] == str(cfg[key]) and word in text, (key, word)
    r = run("bench.py", "--help")
    assert r.returncode == 0 and "--batch" in r.stdout and "--context" in r.stdout


def test_trace_run_and_command_line_show_their_options():
    r = run(os.path.join("bin", "trace_run"), "--help")
    assert r.returncode == 0
    for opt in ("--model", "--dtype", "--out", "--max-tokens"):
        assert opt in r.stdout
    r = run(os.path.join("bin", "allpaca-amd"), "generate", "--help")
    assert r.returncode == 0
    for opt in ("--model", "--synthetic", "--seed", "--dtype", "--prompt-tokens", "--max-tokens", "--temperature",
                "--top-k", "--top-p", "--page-tokens", "--num-pages", "--chunk-tokens", "--max-batch-tokens"):
        assert opt in r.stdout
