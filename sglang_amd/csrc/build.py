"""Build libfp8k.so (hand-written HIP kernels for gfx950 + the C ABI) in-tree with hipcc.

Usage: python sglang_amd/csrc/build.py [--force] [--jobs N]
Each .hip file is compiled to an object next to it and linked into sglang_amd/csrc/libfp8k.so.
"""
from __future__ import annotations

import argparse
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "libfp8k.so")
SOURCES = ["api.hip", "quant.hip", "gemm.hip", "moe.hip", "tune.hip"]
HEADERS = ["fp8k_common.h", "quant_math.h", "gemm_kernels.h", "gemm_direct.h", "gemm_moe256.h", "gemm_tile128.h", os.path.join("..", "..", "include", "fp8k.h"),
           os.path.join("..", "..", "include", "fp8k_tune.h")]

# -packed-fp32-ops off: packed float32 VALU forms are not used on this hardware pool.
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-Wno-unknown-warning-option",
    "-Wno-pass-failed",
]


def hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found; the fp8k library can only be built with the ROCm toolchain")


def _stale(target: str, deps: list[str]) -> bool:
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.exists(d) and os.path.getmtime(d) > t for d in deps)


def _run(cmd: list[str]) -> None:
    p = subprocess.run(cmd, cwd=HERE, capture_output=True, text=True)
    err = "\n".join(l for l in (p.stdout + p.stderr).splitlines() if "not a recognized feature" not in l)
    if p.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), err))
    if err.strip():
        sys.stderr.write(err + "\n")


def build(force: bool = False, jobs: int = 4, verbose: bool = True) -> str:
    cc = hipcc()
    srcs = [s for s in SOURCES if os.path.exists(os.path.join(HERE, s))]
    hdrs = [os.path.join(HERE, h) for h in HEADERS]
    objs = []
    todo = []
    for s in srcs:
        o = os.path.join(HERE, s[:-4] + ".o")
        objs.append(o)
        if force or _stale(o, [os.path.join(HERE, s), os.path.abspath(__file__)] + hdrs):
            todo.append([cc] + FLAGS + ["-c", s, "-o", o])
    if verbose and todo:
        print("[fp8k] compiling %d file(s) for gfx950" % len(todo), flush=True)
    with ThreadPoolExecutor(max_workers=max(1, jobs)) as ex:
        list(ex.map(_run, todo))
    if todo or force or _stale(LIB, objs):
        _run([cc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs)
        if verbose:
            print("[fp8k] linked", LIB, flush=True)
    return LIB


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--force", action="store_true")
    ap.add_argument("--jobs", type=int, default=4)
    a = ap.parse_args()
    build(force=a.force, jobs=a.jobs)
