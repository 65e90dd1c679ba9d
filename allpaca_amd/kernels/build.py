"""Builds the HIP kernel libraries for gfx950 with hipcc and finds them again.

Two kernel libraries, so that a run compiles only what it needs: `plain` (the whole
float32 path and the small steps of the bfloat16 path) and `tuned` (MFMA matrix
products and attention for bfloat16); and `host`, the engine's host side in C++
(plan executor, cache manager, step packer, scheduler), which is linked against both.  Objects and libraries live in
`allpaca_amd/_build/` (or, if the package folder cannot be written, in a
per-user folder under the system's temporary directory).  A library is rebuilt
when the text of its sources or the flags change."""
from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from concurrent.futures import ThreadPoolExecutor
from typing import Dict, List

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")

LIBS: Dict[str, List[str]] = {
    "plain": ["plain_ops.hip", "plain_gemm.hip", "plain_attention.hip", "sampling.hip"],
    "tuned": ["gemm_bf16.hip", "gemm_wide_bf16.hip", "gemm_direct_bf16.hip", "skinny_gemm_bf16.hip", "attention_bf16.hip", "attention_wide_bf16.hip", "rope_bf16.hip"],
    # what measurements need and the engine does not (what a streaming read and a loop of MFMAs reach on this card)
    "bench": ["probe.hip"],
    "host": ["host/exec.cpp", "host/cache.cpp", "host/pack.cpp", "host/sched.cpp"],
}
HEADERS = ["common.h", "mfma.h", "gemm_wide.h", "gemm_direct.h", "attention_wide.h", "no_alloc.h",
           "host/host.h", "host/kernels.h", "host/rules.h", "host/cache.h"]
# libraries a library is linked against (built first; found at run time beside it)
NEEDS: Dict[str, List[str]] = {"host": ["plain", "tuned"]}
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-Wno-unused-value", "-Wno-unused-result"]

ARCH = "gfx950"
# -packed-fp32-ops is switched off for device code: some packed forms have given wrong results on this hardware.
# MFMA accumulators stay in ordinary vector registers (-amdgpu-mfma-vgpr-form): the attention kernels rescale their
# accumulators with vector instructions every step, and from accumulation registers every value would have to be
# moved there and back.
FLAGS = ["-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden", f"--offload-arch={ARCH}",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-mllvm", "-amdgpu-mfma-vgpr-form=1",
         "-Wno-unused-result"]
# Sources whose MFMA accumulators go into the accumulation registers (the compiler's default): a kernel there keeps 256
# of them a wave, beside 256 vector registers for everything else.
ACC_REGISTER_SOURCES = {"gemm_wide_bf16.hip", "gemm_direct_bf16.hip", "attention_wide_bf16.hip"}
VGPR_FORM = ["-mllvm", "-amdgpu-mfma-vgpr-form=1"]


def flags_for(src: str) -> List[str]:
    if src.endswith(".cpp"):      # host code: no device pass
        return list(HOST_FLAGS)
    if os.path.basename(src) not in ACC_REGISTER_SOURCES:
        return list(FLAGS)
    out, skip = [], 0
    for i, f in enumerate(FLAGS):
        if skip:
            skip -= 1
        elif FLAGS[i:i + 2] == VGPR_FORM:
            skip = 1
        else:
            out.append(f)
    return out


class KernelBuildError(RuntimeError):
    pass


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand):
            return cand
    raise KernelBuildError("hipcc not found (looked at $HIPCC, PATH, /opt/rocm/bin/hipcc); "
                           "the engine has no fallback without its HIP kernels")


def build_dir() -> str:
    here = os.path.join(os.path.dirname(CSRC), "_build")
    try:
        os.makedirs(here, exist_ok=True)
        probe = os.path.join(here, f".w{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return here
    except OSError:
        alt = os.path.join(tempfile.gettempdir(), f"allpaca_amd_build_{os.getuid()}")
        os.makedirs(alt, exist_ok=True)
        return alt


def _sources(name: str) -> List[str]:
    return [os.path.join(CSRC, f) for f in LIBS[name]]


def source_hash(name: str) -> str:
    h = hashlib.sha256()
    h.update(" ".join(FLAGS + HOST_FLAGS).encode())
    h.update(" ".join(sorted(ACC_REGISTER_SOURCES)).encode())
    for dep in NEEDS.get(name, []):
        h.update(source_hash(dep).encode())
    for path in _sources(name) + [os.path.join(CSRC, f) for f in HEADERS]:
        if os.path.isfile(path):
            h.update(os.path.basename(path).encode())
            with open(path, "rb") as f:
                h.update(f.read())
    return h.hexdigest()


def lib_path(name: str, directory: str | None = None) -> str:
    return os.path.join(directory or build_dir(), f"liballpaca_{name}.so")


def is_current(name: str) -> bool:
    d = build_dir()
    stamp = os.path.join(d, f"{name}.hash")
    if not (os.path.isfile(lib_path(name, d)) and os.path.isfile(stamp)):
        return False
    with open(stamp) as f:
        return f.read().strip() == source_hash(name)


def _say(msg: str) -> None:
    print(f"[allpaca_amd build] {msg}", file=sys.stderr, flush=True)


def build(name: str, force: bool = False, verbose: bool = True) -> str:
    """Compile library `name`; returns the path of the .so."""
    if name not in LIBS:
        raise KernelBuildError(f"no kernel library {name!r}; known: {sorted(LIBS)}")
    for dep in NEEDS.get(name, []):
        build(dep, force=False, verbose=verbose)
    if not force and is_current(name):
        return lib_path(name)
    hipcc = _hipcc()
    d = build_dir()
    srcs = _sources(name)
    for s in srcs:
        if not os.path.isfile(s):
            raise KernelBuildError(f"kernel source {s} is missing")
    t0 = time.time()
    if verbose:
        _say(f"compiling library '{name}' ({len(srcs)} files) for {ARCH} into {d}")
    done = threading.Event()

    def ticker():
        while not done.wait(20.0):
            _say(f"... still compiling '{name}' ({time.time() - t0:.0f} s)")

    if verbose:
        threading.Thread(target=ticker, daemon=True).start()

    def compile_one(src: str) -> str:
        # names of this process only: two processes may build the same library into the same folder at once
        obj = os.path.join(d, f"{name}_{os.path.splitext(os.path.basename(src))[0]}.{os.getpid()}.o")
        cmd = [hipcc, *flags_for(src), "-I", CSRC, "-c", src, "-o", obj]
        p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if p.returncode != 0:
            raise KernelBuildError(f"hipcc failed on {src}:\n{p.stdout}")
        if verbose:
            _say(f"compiled {os.path.basename(src)} ({time.time() - t0:.0f} s)")
        return obj

    objs: List[str] = []
    try:
        workers = max(1, min(len(srcs), os.cpu_count() or 1, 8))
        with ThreadPoolExecutor(workers) as ex:
            objs = list(ex.map(compile_one, srcs))
        out = lib_path(name, d)
        tmp = out + f".tmp{os.getpid()}"
        deps = [f"-lallpaca_{dep}" for dep in NEEDS.get(name, [])]
        if deps:
            deps = ["-L", d, *deps, "-Wl,-rpath,$ORIGIN"]
        p = subprocess.run([hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", *objs, *deps, "-o", tmp],
                           stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if p.returncode != 0:
            raise KernelBuildError(f"link of {out} failed:\n{p.stdout}")
        os.replace(tmp, out)
        stamp = os.path.join(d, f"{name}.hash")
        with open(stamp + f".tmp{os.getpid()}", "w") as f:
            f.write(source_hash(name))
        os.replace(stamp + f".tmp{os.getpid()}", stamp)
    finally:
        done.set()
        for src in srcs:
            obj = os.path.join(d, f"{name}_{os.path.splitext(os.path.basename(src))[0]}.{os.getpid()}.o")
            if os.path.isfile(obj):
                os.remove(obj)
    if verbose:
        _say(f"library '{name}' ready in {time.time() - t0:.0f} s")
    return out


def build_all(force: bool = True, verbose: bool = True) -> List[str]:
    return [build(n, force=force, verbose=verbose) for n in LIBS]   # (in the order of LIBS: what is needed comes first)
