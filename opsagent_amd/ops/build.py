"""Build the HIP kernel library for gfx950 (MI355X) — in-tree, so the .so
travels with the repo snapshot to GPU boxes.

Usage: python -m opsagent_amd.ops.build [--check]
Called by __graft_entry__.build().
"""

from __future__ import annotations

import os
import subprocess
import sys

CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libopsagent_kernels.so")

SOURCES = [
    "rmsnorm.hip",
    "gemv.hip",
    "rope.hip",
    "rope_kv.hip",
    "elementwise.hip",
    "sampling.hip",
    "attention_decode.hip",
    "attention_prefill.hip",
    "fp8_moe.hip",
    "moe_gemv.hip",
]

# the sequence-mixer kernels of hybrid decoders live in a library of their
# own: a checkout that serves only such a model compiles just what it loads
MIXER_SOURCES = ["mixers.hip", "blocks.hip", "prenorm.hip", "recurrent.hip", "hyper.hip"]
MIXER_OUT = os.path.join(
    os.path.dirname(os.path.abspath(__file__)), "libopsagent_mixers.so"
)

# packed-fp32 VALU forms are switched off for every kernel
HIP_FLAGS = ["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]

HIPCC = os.environ.get("HIPCC", "hipcc")
ARCH = os.environ.get("OPSAGENT_GPU_ARCH", "gfx950")

GRAMMAR_OUT = os.path.join(
    os.path.dirname(os.path.abspath(__file__)), "libopsagent_grammar.so"
)
GRAMMAR_SRC = os.path.join(CSRC, "grammar_fsm.cpp")


def _mtime(path: str) -> float:
    try:
        return os.path.getmtime(path)
    except OSError:
        return 0.0


def needs_rebuild(out: str = OUT, sources=None) -> bool:
    out_t = _mtime(out)
    if out_t == 0.0:
        return True
    deps = [os.path.join(CSRC, s) for s in (sources or SOURCES)]
    deps.append(os.path.join(CSRC, "common.h"))
    deps.append(os.path.join(CSRC, "mixer_util.h"))
    return any(_mtime(d) > out_t for d in deps)


def _compile_library(sources, out: str, verbose: bool) -> str:
    """Compile each source to an object (in parallel), then link. The
    library is written under a temporary name and renamed into place, so a
    concurrent process never loads a half-written file."""
    import tempfile
    from concurrent.futures import ThreadPoolExecutor

    tmp = tempfile.mkdtemp(prefix="opsagent_build_")
    base = [HIPCC, f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", *HIP_FLAGS]

    def one(src: str) -> str:
        obj = os.path.join(tmp, src + ".o")
        cmd = base + ["-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print("[opsagent build]", " ".join(cmd), file=sys.stderr)
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError(
                f"hipcc failed ({proc.returncode}) on {src}:\n{proc.stdout}\n{proc.stderr}"
            )
        return obj

    try:
        jobs = max(1, min(len(sources), int(os.environ.get("MAX_JOBS", "8"))))
        with ThreadPoolExecutor(jobs) as pool:
            objs = list(pool.map(one, sources))
        part = out + f".{os.getpid()}.part"
        cmd = [HIPCC, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", part, *objs]
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"link failed ({proc.returncode}):\n{proc.stdout}\n{proc.stderr}")
        os.replace(part, out)
    finally:
        import shutil

        shutil.rmtree(tmp, ignore_errors=True)
    return out


def build(verbose: bool = True, force: bool = False) -> str:
    if not force and not needs_rebuild():
        return OUT
    return _compile_library(SOURCES, OUT, verbose)


def build_mixers(verbose: bool = True, force: bool = False) -> str:
    if not force and not needs_rebuild(MIXER_OUT, MIXER_SOURCES):
        return MIXER_OUT
    return _compile_library(MIXER_SOURCES, MIXER_OUT, verbose)


def build_grammar(verbose: bool = True, force: bool = False) -> str:
    """Build the CPU grammar-FSM library (plain g++; used on CPU and GPU)."""
    if not force and _mtime(GRAMMAR_OUT) > _mtime(GRAMMAR_SRC):
        return GRAMMAR_OUT
    cmd = ["g++", "-O2", "-std=c++17", "-shared", "-fPIC", "-o", GRAMMAR_OUT, GRAMMAR_SRC]
    if verbose:
        print("[opsagent build]", " ".join(cmd), file=sys.stderr)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"g++ failed ({proc.returncode}):\n{proc.stderr}")
    return GRAMMAR_OUT


def build_all(force: bool = False) -> None:
    build_grammar(force=force)
    build(force=force)
    build_mixers(force=force)


if __name__ == "__main__":
    build_all(force="--force" in sys.argv)
    print(OUT)
    print(MIXER_OUT)
    print(GRAMMAR_OUT)
