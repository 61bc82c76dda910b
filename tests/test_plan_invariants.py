"""The launch planner (atex_amd/csrc/plan.h) is pure host code: tests/plan_check.cc sweeps it
over about two million shapes (LayerNorm and both InstanceNorm layouts, several CU counts) and
checks every plan against what the kernels and launchers assume of it: rows covered by the lanes
they are given, launch bounds, grid limits, workspace sections large enough for what the kernels
write there, 32-bit positions inside slabs and partials.  No GPU involved."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(os.path.dirname(HERE), "atex_amd", "csrc")


def test_every_plan_satisfies_the_kernels_assumptions(tmp_path):
    exe = str(tmp_path / "plan_check")
    subprocess.run(["g++", "-O1", "-std=c++17", "-I", CSRC, os.path.join(HERE, "plan_check.cc"), "-o", exe],
                   check=True, capture_output=True, text=True)
    run = subprocess.run([exe], capture_output=True, text=True)
    assert run.returncode == 0, run.stdout[-4000:]
    assert run.stdout.startswith("ok ")
    assert int(run.stdout.split()[1]) > 1_000_000
