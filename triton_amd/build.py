"""Builds `libtriton_amd.so` (gfx950 code objects + the C ABI) in-tree with hipcc.

Usage: `python -m triton_amd.build` (or `__graft_entry__.build()`).  hipcc cross-compiles for gfx950
on a machine without a GPU; the shared library lands next to this file and is what `_native.py` loads.
"""
from __future__ import annotations

import concurrent.futures
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libtriton_amd.so")

HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"

# -packed-fp32-ops is switched off for every translation unit of this library.
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def _compile(src: str, force: bool) -> str:
    obj = os.path.join(OBJ, src[:-4] + ".o")
    src_path = os.path.join(CSRC, src)
    if not force and os.path.exists(obj):
        deps = [src_path] + [os.path.join(CSRC, h) for h in os.listdir(CSRC) if h.endswith(".h")]
        deps.append(os.path.join(HERE, "..", "include", "triton_amd.h"))
        if all(os.path.getmtime(d) <= os.path.getmtime(obj) for d in deps):
            return obj
    cmd = [HIPCC, *FLAGS, "-c", src_path, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{r.stdout}\n{r.stderr}")
    warn = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l and l.strip())
    if "warning" in warn:
        sys.stderr.write(warn + "\n")
    return obj


def build(force: bool = True, jobs: int = 8) -> str:
    os.makedirs(OBJ, exist_ok=True)
    srcs = sources()
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(jobs, len(srcs))) as ex:
        objs = list(ex.map(lambda s: _compile(s, force), srcs))
    tmp = LIB + ".tmp"
    r = subprocess.run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", tmp], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    os.replace(tmp, LIB)
    return LIB


if __name__ == "__main__":
    print(build(force="--incremental" not in sys.argv))
