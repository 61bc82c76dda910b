"""The TensorFlow-ROCm op library under tf/ (op registrations, OpKernels, functor
specialisations, Python package) cannot be built or run here: TensorFlow is not installed.
What can be checked without it is that the sources parse and type-check -- above all that every
call into include/atex_norms.h has the right arity and argument types -- against
tests/tf_mock/, a declaration-only stand-in for the few TensorFlow types they use.  This is a
signature check of the glue, not parity evidence: nothing is linked or executed.
"""
import os
import py_compile
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TF = os.path.join(ROOT, "tf")
FLAGS = ["g++", "-fsyntax-only", "-std=c++17", "-Wall", "-Wextra", "-Werror", "-I", os.path.join(ROOT, "include"),
         "-I", TF, "-I", os.path.join(ROOT, "tests", "tf_mock")]


@pytest.mark.parametrize("source,defines", [
    ("norm_ops_rocm.cc", []),
    ("norm_kernels_rocm.cc", []),
    ("fused_norm_functors_rocm.cc", []),
    ("fused_norm_functors_rocm.cc", ["-DATEXN_TF_CPU_FUNCTORS"]),
])
def test_tf_sources_type_check_against_the_mock(source, defines):
    r = subprocess.run(FLAGS + defines + [os.path.join(TF, source)], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr


def test_a_wrong_call_into_the_c_abi_is_caught(tmp_path):
    """The check has teeth: the same file with one argument dropped from a library call fails."""
    src = open(os.path.join(TF, "fused_norm_functors_rocm.cc")).read()
    broken = src.replace("ws.ptr(), ws.bytes(), StreamOf(ctx))));", "ws.ptr(), StreamOf(ctx))));", 1)
    assert broken != src
    p = tmp_path / "broken.cc"
    p.write_text(broken)
    r = subprocess.run(FLAGS + [str(p)], capture_output=True, text=True)
    assert r.returncode != 0 and "atexn_layer_norm_fwd" in r.stderr


def test_tf_python_package_compiles_and_needs_tensorflow():
    for f in ("__init__.py", "ops.py"):
        py_compile.compile(os.path.join(TF, "nv_norms", f), doraise=True)
    text = open(os.path.join(TF, "nv_norms", "ops.py")).read()
    # tensorflow_addons only inside InstanceNormalization.__init__
    assert text.count("import tensorflow_addons") == 1
    assert text.index("import tensorflow_addons") > text.index("class InstanceNormalization")


def test_cmake_configures_to_nothing_without_tensorflow(tmp_path):
    import importlib.util

    if importlib.util.find_spec("tensorflow") is not None:
        pytest.skip("TensorFlow is installed: the real build applies")
    r = subprocess.run(["cmake", "-S", TF, "-B", str(tmp_path)], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    assert "the op library is not built" in r.stdout
