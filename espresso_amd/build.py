"""Builds libespresso_hip.so for gfx950 with hipcc (cross-compiles without a GPU).

Every source is compiled to an object of its own, several at a time, and the objects are linked into the shared
library.  build() recompiles everything; build(incremental=True) keeps objects that are newer than their source and
every header (a convenience while developing).
"""
from __future__ import annotations

import glob
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
OBJ_DIR = os.path.join(HERE, "build")
LIB_PATH = os.path.join(LIB_DIR, "libespresso_hip.so")

# -packed-fp32-ops is switched off on purpose: packed fp32 VALU forms are not used in this library.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-mllvm", "-amdgpu-kernarg-preload-count=14",
    "-Wall", "-Wno-unused-function", "-Wno-c++20-extensions",   # templated lambdas (compile-time piece indices in gemm_split.hip)
]
NOISE = "is not a recognized feature for this target"


def sources() -> list[str]:
    return sorted(glob.glob(os.path.join(CSRC, "*.cpp")) + glob.glob(os.path.join(CSRC, "host", "*.cpp")) +
                  glob.glob(os.path.join(CSRC, "kernels", "*.hip")))


def headers() -> list[str]:
    return (glob.glob(os.path.join(CSRC, "**", "*.h"), recursive=True) +
            glob.glob(os.path.join(HERE, "..", "include", "*.h")))


def _object_path(src: str) -> str:
    return os.path.join(OBJ_DIR, os.path.relpath(src, CSRC).replace(os.sep, "__") + ".o")


def _run(cmd: list[str]) -> str:
    proc = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in proc.stderr.splitlines() if NOISE not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed: {' '.join(cmd)}\n{err}")
    return err


def build(verbose: bool = False, incremental: bool = False, jobs: int = 8) -> str:
    os.makedirs(LIB_DIR, exist_ok=True)
    os.makedirs(OBJ_DIR, exist_ok=True)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    newest_header = max(os.path.getmtime(h) for h in headers())
    todo = []
    for src in sources():
        obj = _object_path(src)
        fresh = incremental and os.path.exists(obj) and os.path.getmtime(obj) > max(os.path.getmtime(src), newest_header)
        if not fresh:
            todo.append([hipcc, *HIPCC_FLAGS, "-I", os.path.join(HERE, "..", "include"), "-c", "-x", "hip", src, "-o", obj])
    with ThreadPoolExecutor(max_workers=max(1, jobs)) as pool:
        for cmd, err in zip(todo, pool.map(_run, todo)):
            if verbose:
                print(" ".join(cmd))
                if err.strip():
                    print(err, file=sys.stderr)
    err = _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *[_object_path(s) for s in sources()]])
    if verbose and err.strip():
        print(err, file=sys.stderr)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv, incremental="--incremental" in sys.argv))
