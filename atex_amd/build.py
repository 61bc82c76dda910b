"""Builds libatex_norms_hip.so in-tree with hipcc for gfx950.

    python -m atex_amd.build [--force]

Each .hip translation unit is compiled to an object (in parallel), then linked into
atex_amd/lib/libatex_norms_hip.so.  No CMake, no torch: the library depends only on the HIP
runtime.
"""
from __future__ import annotations

import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(HERE, "build")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libatex_norms_hip.so")

SOURCES = [
    "capi.hip",
    "dispatch.hip",
    "rows_launch_f32.hip",
    "rows_launch_f16.hip",
    "rows_launch_bf16.hip",
    "cl_launch.hip",
]

# -packed-fp32-ops off: hipcc must not form v_pk_*_f32 from ordinary float code.
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-gpu-rdc",
    "-Wall",
    "-Wno-unused-function",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def _deps_mtime() -> float:
    m = 0.0
    for f in os.listdir(CSRC):
        if f.endswith((".cuh", ".h")):
            m = max(m, os.path.getmtime(os.path.join(CSRC, f)))
    m = max(m, os.path.getmtime(os.path.join(HERE, "..", "include", "atex_norms.h")))
    return m


def _compile(src: str, force: bool, dep_m: float) -> str:
    obj = os.path.join(OBJ_DIR, src.replace(".hip", ".o"))
    s = os.path.join(CSRC, src)
    if not force and os.path.exists(obj) and os.path.getmtime(obj) >= max(os.path.getmtime(s), dep_m):
        return obj
    cmd = [_hipcc(), *HIPCC_FLAGS, "-c", s, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(force: bool = False, jobs: int = 6) -> str:
    os.makedirs(OBJ_DIR, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    dep_m = _deps_mtime()
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, force, dep_m), SOURCES))
    if force or not os.path.exists(LIB_PATH) or any(os.path.getmtime(o) > os.path.getmtime(LIB_PATH) for o in objs):
        cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", *objs, "-o", LIB_PATH]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("link failed:\n" + r.stderr)
    return LIB_PATH


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
