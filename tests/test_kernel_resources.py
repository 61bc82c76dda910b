"""The compiler's account of every kernel of the product library, held to a budget.

`python -m atex_amd.build` writes atex_amd/lib/kernel_resources.json from hipcc's
-Rpass-analysis=kernel-resource-usage remarks (registers, bytes of scratch memory per lane,
spilled registers).  A kernel that starts to spill does not fail any parity test, it only gets
slow: the bf16 build of a kernel written against fp16 once kept 64 converted floats beside the raw
vectors and spilled 98 registers under a launch bound that fp16 met, 2.5 times the fp16 duration.
No GPU is needed: the figures are the compiler's."""
import json
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REPORT = os.path.join(ROOT, "atex_amd", "lib", "kernel_resources.json")

# Kernels that may keep a few registers in scratch memory, and why.  (pattern on the mangled name,
# most spilled registers allowed)
ALLOWED = [
    # builds for more workgroups per CU: the bound is the point, the spills were measured to pay
    (r"13cl_fwd_singleI.*Lb1EEEv", 12),
    (r"13cl_bwd_singleI.*Lb1ELb1EEEv", 20),
    (r"16plane_bwd_singleI.*Lb1ELb1EEEv", 12),
    # sixteen pixels per thread of a ragged channel vector, channels that are no multiple of a vector
    (r"12cl_fwd_applyI.*Li16E", 20),
    # rows that are not vector-aligned, accumulators in LDS
    (r"12rows_bwd_ldsI", 14),
    # a value or two kept for a path that is seldom taken
    (r"17rows_bwd_residentI", 2),
]
HARD_LIMIT = 20

# The kernels of the benchmark configurations: nothing in scratch memory at all.
HOT = [
    "17rows_fwd_residentIDF16_Li8ELi64ELi2ELi2ELb1ELb0ELb0EE",  # LN [8192, 1024] fp16 forward
    "17rows_bwd_residentIDF16_Li8ELi64ELi2ELi1ELb1ELb0ELb0EE",  # ... backward
    "17rows_bwd_residentIDF16_Li8ELi0ELi4ELi1ELb1ELb1ELb0EE",   # IN [8, 64, 128, 128] channel-first backward
    "13cl_fwd_singleIDF16_Li8ELi8ELb1ELb0EE",                   # IN [8, 128, 128, 64] channels-last
    "13cl_bwd_singleIDF16_Li8ELi8ELb1ELb0EE",
    "16plane_fwd_singleIDF16_Li8ELi8ELb1ELb1EE",                # IN [2, 32, 128^3] channel-first
    "16plane_fwd_singleIDF16bLi8ELi8ELb1ELb1EE",                # ... in bf16
    "12cl_fwd_statsIDF16_Li8ELi0E", "11cl_bwd_sumsIDF16_Li8ELi0E",  # IN [2, 128^3, 32] channels-last
    "12cl_fwd_applyIDF16_Li8ELi0E", "12cl_bwd_applyIDF16_Li8ELi0E",
]


@pytest.fixture(scope="module")
def kernels():
    if not os.path.exists(REPORT):
        pytest.skip("no kernel_resources.json: run python -m atex_amd.build")
    with open(REPORT) as f:
        per_unit = json.load(f)
    merged = {}
    for unit, ks in per_unit.items():
        for name, r in ks.items():
            merged[name] = dict(r, unit=unit)
    return merged


def test_the_report_covers_the_library(kernels):
    units = {r["unit"] for r in kernels.values()}
    assert {"rows_launch_f32", "rows_launch_f16", "rows_launch_bf16", "cl_launch", "dispatch"} <= units
    assert len(kernels) > 1000
    for name, r in kernels.items():
        assert {"vgprs", "sgprs", "scratch_bytes_per_lane", "vgpr_spills", "waves_per_simd"} <= set(r), name


def test_no_kernel_spills_beyond_its_allowance(kernels):
    over = []
    for name, r in kernels.items():
        spills = r["vgpr_spills"]
        if spills == 0:
            continue
        allowance = max([limit for pat, limit in ALLOWED if re.search(pat, name)], default=0)
        if spills > min(allowance, HARD_LIMIT):
            over.append(f"{name}: {spills} registers spilled ({r['vgprs']} VGPRs), allowance {allowance}")
    assert not over, "\n".join(over)


def test_the_configurations_kernels_use_no_scratch_memory(kernels):
    for frag in HOT:
        hits = [n for n in kernels if frag in n]
        assert hits, f"no kernel matches {frag}: has an instantiation been renamed?"
        for n in hits:
            assert kernels[n]["scratch_bytes_per_lane"] == 0, f"{n}: {kernels[n]}"


def test_bf16_builds_need_no_more_scratch_than_fp16_plus_a_little(kernels):
    """bf16 has no mixed-precision arithmetic (conversions cost registers); a twin far above its
    fp16 kernel means the code keeps converted copies alive."""
    worse = []
    for name, r in kernels.items():
        if "DF16_" not in name:
            continue
        twin = kernels.get(name.replace("DF16_", "DF16b"))
        if twin is None:
            continue
        if twin["vgpr_spills"] > r["vgpr_spills"] + 8:
            worse.append(f"{name}: fp16 spills {r['vgpr_spills']}, bf16 {twin['vgpr_spills']}")
    assert not worse, "\n".join(worse)
