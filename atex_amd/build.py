"""Builds libatex_norms_hip.so in-tree with hipcc for gfx950.

    python -m atex_amd.build [--force] [--product-only]

Each .hip translation unit is compiled to an object (in parallel), then linked into
atex_amd/lib/libatex_norms_hip.so.  No CMake, no torch: the library depends only on the HIP
runtime.

A second library, libatex_norms_hip_bench.so, is the same sources compiled with
-DATEXN_BENCH_BUILD: it adds the entry points of csrc/bench_hooks.h (launch-planning switches,
a plan description), which bench.py and the tests that force a kernel family use.

The compiler's account of every kernel of the product library (registers, bytes of scratch
memory per lane, spilled registers, occupancy) is written to lib/kernel_resources.json, which
tests/test_kernel_resources.py holds to a budget: a kernel that quietly starts to spill is a
kernel that has become slow.
"""
from __future__ import annotations

import concurrent.futures
import json
import os
import re
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(HERE, "build")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libatex_norms_hip.so")
BENCH_LIB_PATH = os.path.join(LIB_DIR, "libatex_norms_hip_bench.so")
RESOURCES_PATH = os.path.join(LIB_DIR, "kernel_resources.json")

SOURCES = [
    "capi.hip",
    "dispatch.hip",
    "rows_launch_f32.hip",
    "rows_launch_f16.hip",
    "rows_launch_bf16.hip",
    "cl_launch.hip",
    "cpu_kernels.cc",
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
        if f.endswith(".h"):
            m = max(m, os.path.getmtime(os.path.join(CSRC, f)))
    m = max(m, os.path.getmtime(os.path.join(HERE, "..", "include", "atex_norms.h")))
    return m


def _compile(src: str, force: bool, dep_m: float, bench: bool) -> str:
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ("_bench.o" if bench else ".o"))
    s = os.path.join(CSRC, src)
    if not force and os.path.exists(obj) and os.path.getmtime(obj) >= max(os.path.getmtime(s), dep_m):
        return obj
    report = not bench and src.endswith(".hip")
    cmd = [_hipcc(), *HIPCC_FLAGS, *(["-DATEXN_BENCH_BUILD"] if bench else []),
           *(["-Rpass-analysis=kernel-resource-usage"] if report else []), "-c", s, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    lines = [l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l]
    if report:
        with open(obj + ".resources.json", "w") as f:
            json.dump(_kernel_resources(lines), f)
        lines = _without_remarks(lines)
    err = "\n".join(lines)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


_REMARK = "[-Rpass-analysis=kernel-resource-usage]"
_FIELDS = {"TotalSGPRs": "sgprs", "VGPRs": "vgprs", "ScratchSize [bytes/lane]": "scratch_bytes_per_lane",
           "Occupancy [waves/SIMD]": "waves_per_simd", "SGPRs Spill": "sgpr_spills", "VGPRs Spill": "vgpr_spills",
           "LDS Size [bytes/block]": "lds_bytes"}


def _kernel_resources(stderr_lines) -> dict:
    """{mangled kernel name: {vgprs, sgprs, scratch_bytes_per_lane, vgpr_spills, ...}} from the
    remarks of -Rpass-analysis=kernel-resource-usage."""
    out, cur = {}, None
    for l in stderr_lines:
        if _REMARK not in l:
            continue
        m = re.search(r"remark:\s+(.*?):\s+(\S+)\s+\[-Rpass", l)
        if not m:
            continue
        key, val = m.group(1).strip(), m.group(2)
        if key == "Function Name":
            cur = out.setdefault(val, {})
        elif cur is not None and key in _FIELDS:
            cur[_FIELDS[key]] = int(val)
    return out


def _without_remarks(lines):
    """Drops the remarks and the source excerpts that clang prints under them."""
    kept, skip = [], 0
    for l in lines:
        if _REMARK in l:
            skip = 2  # the quoted source line and its caret line, when present
            continue
        if skip and (re.match(r"\s*\d+ \| ", l) or re.match(r"\s*\| ", l)):
            skip -= 1
            continue
        skip = 0
        if l.startswith("In file included from"):
            continue
        kept.append(l)
    return kept


def _link(objs, path: str, force: bool) -> None:
    if force or not os.path.exists(path) or any(os.path.getmtime(o) > os.path.getmtime(path) for o in objs):
        cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", *objs, "-o", path]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("link failed:\n" + r.stderr)


def build(force: bool = False, jobs: int = 8, bench: bool = True) -> str:
    """Compiles the product library and (bench=True) the benchmark variant."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    dep_m = _deps_mtime()
    units = [(s, False) for s in SOURCES] + ([(s, True) for s in SOURCES] if bench else [])
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda u: _compile(u[0], force, dep_m, u[1]), units))
    _link(objs[:len(SOURCES)], LIB_PATH, force)
    merged = {}
    for o in objs[:len(SOURCES)]:
        if os.path.exists(o + ".resources.json"):
            with open(o + ".resources.json") as f:
                merged[os.path.basename(o)[:-2]] = json.load(f)
    with open(RESOURCES_PATH, "w") as f:
        json.dump(merged, f, indent=0, sort_keys=True)
    if bench:
        _link(objs[len(SOURCES):], BENCH_LIB_PATH, force)
    return LIB_PATH


if __name__ == "__main__":
    print(build(force="--force" in sys.argv, bench="--product-only" not in sys.argv))
