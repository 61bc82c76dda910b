"""Host logic of the ops through the C ABI, no GPU needed: axis packing, data_format
parsing, flattening, argument validation (every check precedes any launch), the exported
symbol set and the workspace queries.  Sources: cc/ops/norm_ops.cc:18-144,
cc/kernels/fused_layer_norm_op.cc:252-458, cc/kernels/fused_instance_norm_op.cc:25-534 and
the axis cases of tests/fused_layer_norm_test.py:250-260."""
import ctypes
import os
import re
import subprocess

import pytest

from atex_amd.nv_norms import _capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def L():
    return _capi.lib()


def resolve_axes(L, dims, axis):
    d = (ctypes.c_int64 * len(dims))(*dims)
    a = (ctypes.c_int * max(len(axis), 1))(*axis)
    n, dd = ctypes.c_int64(), ctypes.c_int64()
    st = L.atexn_layer_norm_resolve_axes(len(dims), d, a, len(axis), ctypes.byref(n), ctypes.byref(dd))
    return st, n.value, dd.value, L.atexn_last_error().decode()


def resolve_format(L, dims, fmt):
    d = (ctypes.c_int64 * len(dims))(*dims)
    lay = ctypes.c_int()
    n, c, dd = ctypes.c_int64(), ctypes.c_int64(), ctypes.c_int64()
    st = L.atexn_instance_norm_resolve_format(len(dims), d, fmt, ctypes.byref(lay), ctypes.byref(n),
                                              ctypes.byref(c), ctypes.byref(dd))
    return st, lay.value, n.value, c.value, dd.value, L.atexn_last_error().decode()


def test_every_declared_symbol_is_exported(L):
    header = open(os.path.join(ROOT, "include", "atex_norms.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    names = sorted(set(re.findall(r"\b(atexn_[a-z0-9_]+)\s*\(", header)))
    assert len(names) >= 19, names
    for n in names:
        assert hasattr(L, n), f"{n} is declared in atex_norms.h but not exported"
    assert set(names) <= set(_capi.SIGNATURES), set(names) - set(_capi.SIGNATURES)
    # and nothing beyond the header: every exported atexn_* symbol of the product library is
    # declared there; its benchmark variant adds exactly what csrc/bench_hooks.h declares (the
    # process-wide tuning switch among them, which the product library must not have)
    hooks = open(os.path.join(ROOT, "atex_amd", "csrc", "bench_hooks.h")).read()
    hooks = re.sub(r"/\*.*?\*/", "", hooks, flags=re.S)
    hook_names = set(re.findall(r"\b(atexn_[a-z0-9_]+)\s*\(", hooks))
    assert hook_names == set(_capi.BENCH_SIGNATURES) and "atexn_set_tuning" in hook_names
    for path, want in ((_capi.LIB_PATH, set(names)), (_capi.BENCH_LIB_PATH, set(names) | hook_names)):
        out = subprocess.run(["nm", "-D", "--defined-only", path], capture_output=True, text=True, check=True).stdout
        exported = {line.split()[-1] for line in out.splitlines() if line.split()[-1].startswith("atexn_")}
        assert exported == want, (path, exported ^ want)
    assert L.atexn_abi_version() == 2
    assert L.atexn_status_string(0) == b"OK"
    assert L.atexn_status_string(1) == b"INVALID_ARGUMENT"
    assert L.atexn_status_string(2) == b"LAUNCH_ERROR"


@pytest.mark.parametrize("dims,axis,N,D", [
    ((2, 3, 4), [1, 2], 2, 12), ((2, 3, 4), [-2, -1], 2, 12), ((2, 3, 4), [1, -1], 2, 12),
    ((2, 3, 4), [-2, 2], 2, 12), ((2, 3, 4), [-1], 6, 4), ((2, 3, 4), [2], 6, 4),
    ((2, 3, 4), [2, 2, -1], 6, 4),                       # duplicates are removed
    ((2, 3, 4), [0, 1, 2], 1, 24), ((7,), [0], 1, 7), ((12000, 128, 8, 8), [1, 2, 3], 12000, 8192),
    ((0, 0), [-1], 0, 0), ((5, 0), [-1], 5, 0),
])
def test_layer_norm_axis_packing(L, dims, axis, N, D):
    st, n, d, msg = resolve_axes(L, dims, axis)
    assert st == 0, msg
    assert (n, d) == (N, D)


@pytest.mark.parametrize("dims,axis,needle", [
    ((2, 3, 4), [1], "axis is not packed from last dim."),
    ((2, 3, 4), [0, 2], "axis is not packed from last dim."),
    ((2, 3, 4), [3], "axis contains invalid value: 3"),
    ((2, 3, 4), [-4], "axis contains invalid value: -4"),
    ((2, 3, 4), [], "axis must not be empty"),
])
def test_layer_norm_axis_errors(L, dims, axis, needle):
    st, _, _, msg = resolve_axes(L, dims, axis)
    assert st == _capi.ATEXN_INVALID_ARGUMENT
    assert needle in msg


@pytest.mark.parametrize("fmt,dims,layout,N,C,D", [
    (b"NC...", (2, 32, 8, 8), 0, 2, 32, 64), (b"N...C", (2, 8, 8, 32), 1, 2, 32, 64),
    (b"NCHW", (2, 32, 8, 8), 0, 2, 32, 64), (b"NHWC", (2, 8, 8, 32), 1, 2, 32, 64),
    (b"NCDHW", (2, 32, 4, 8, 8), 0, 2, 32, 256), (b"NDHWC", (2, 4, 8, 8, 32), 1, 2, 32, 256),
    (None, (2, 4, 8, 8, 32), 1, 2, 32, 256),             # attr missing: channels-last
    (b"NCC", (2, 3, 4, 5), 0, 2, 3, 20),                 # a 'C' in position 1 wins
    (b"NC...", (0, 0, 0, 0, 0), 0, 0, 0, 0),
])
def test_instance_norm_format(L, fmt, dims, layout, N, C, D):
    st, lay, n, c, d, msg = resolve_format(L, dims, fmt)
    assert st == 0, msg
    assert (lay, n, c, d) == (layout, N, C, D)


@pytest.mark.parametrize("fmt,dims,needle", [
    (b"NHW", (2, 8, 8, 32), "We only accept 'NC...' or 'N...C' data format"),
    (b"CHWN", (2, 8, 8, 32), "We only accept"),
    (b"NC", (2, 8, 8, 32), "We only accept"),
    (b"", (2, 8, 8, 32), "We only accept"),
    (b"NHWC", (2, 8, 32), "input must be at least 4-dimensional"),
])
def test_instance_norm_format_errors(L, fmt, dims, needle):
    st, *_, msg = resolve_format(L, dims, fmt)
    assert st == _capi.ATEXN_INVALID_ARGUMENT
    assert needle in msg


FAKE = 0x1000  # a non-NULL "device pointer"; every case below is rejected before any launch


def T(dtype, shape, ptr=FAKE):
    return _capi.make_tensor(dtype, shape, ptr)


def call_ln(L, x, scale, offset, axis, y, m, r):
    ax = (ctypes.c_int * len(axis))(*axis)
    st = L.atexn_fused_layer_norm(ctypes.byref(x), ctypes.byref(scale), ctypes.byref(offset), 1e-3, ax,
                                  len(axis), ctypes.byref(y), ctypes.byref(m), ctypes.byref(r), None, 0, None)
    return st, L.atexn_last_error().decode()


def test_fused_layer_norm_validation(L):
    F32, F16 = _capi.ATEXN_F32, _capi.ATEXN_F16
    x = T(F16, (4, 6, 8))
    ok_y, ok_m = T(F16, (4, 6, 8)), T(F32, (4,))
    st, msg = call_ln(L, x, T(F32, (6, 8)), T(F32, (47,)), [1, 2], ok_y, ok_m, ok_m)
    assert st == 1 and "offset must have the same number of elements as the features of x, got 47 and 48" in msg
    st, msg = call_ln(L, x, T(F32, (6, 7)), T(F32, (48,)), [1, 2], ok_y, ok_m, ok_m)
    assert st == 1 and "scale must have the same number of elements" in msg
    st, msg = call_ln(L, x, T(F16, (48,)), T(F32, (48,)), [1, 2], ok_y, ok_m, ok_m)
    assert st == 1 and "must be float32" in msg
    st, msg = call_ln(L, x, T(F32, (48,)), T(F32, (48,)), [1, 2], T(F32, (4, 6, 8)), ok_m, ok_m)
    assert st == 1 and "y must have the dtype and shape of x" in msg
    st, msg = call_ln(L, x, T(F32, (48,)), T(F32, (48,)), [1, 2], ok_y, T(F32, (5,)), ok_m)
    assert st == 1 and "reserve spaces must be rank 1 with 4 elements" in msg
    st, msg = call_ln(L, x, T(F32, (48,)), T(F32, (48,)), [1], ok_y, ok_m, ok_m)
    assert st == 1 and "axis is not packed" in msg
    st, msg = call_ln(L, T(F16, (4, 6, 8), 0), T(F32, (48,)), T(F32, (48,)), [1, 2], ok_y, ok_m, ok_m)
    assert st == 1 and "NULL data pointer" in msg
    st, msg = call_ln(L, T(7, (4, 6, 8)), T(F32, (48,)), T(F32, (48,)), [1, 2], T(7, (4, 6, 8)), ok_m, ok_m)
    assert st == 1 and "bad dtype" in msg
    # empty input: success, nothing launched (fused_layer_norm_test.py:153-164)
    e = T(F32, (0, 0), 0)
    st, msg = call_ln(L, e, T(F32, (0,), 0), T(F32, (0,), 0), [-1], T(F32, (0, 0), 0), T(F32, (0,), 0), T(F32, (0,), 0))
    assert st == 0, msg


def test_fused_layer_norm_grad_validation(L):
    F32 = _capi.ATEXN_F32
    x, dy = T(F32, (4, 8)), T(F32, (4, 8))
    ax = (ctypes.c_int * 1)(-1)

    def call(dy_, x_, scale, m, r, dx, dg, db):
        st = L.atexn_fused_layer_norm_grad(ctypes.byref(dy_), ctypes.byref(x_), ctypes.byref(scale),
                                           ctypes.byref(m), ctypes.byref(r), ax, 1, ctypes.byref(dx),
                                           ctypes.byref(dg), ctypes.byref(db), None, 0, None)
        return st, L.atexn_last_error().decode()

    g, m = T(F32, (8,)), T(F32, (4,))
    st, msg = call(T(F32, (4, 7)), x, g, m, m, T(F32, (4, 8)), g, g)
    assert st == 1 and "x and y_backprop must have same shape" in msg
    st, msg = call(dy, x, g, T(F32, (4, 1)), m, T(F32, (4, 8)), g, g)
    assert st == 1 and "saved mean must be 1-dimensional" in msg
    st, msg = call(dy, x, g, m, T(F32, (3,)), T(F32, (4, 8)), g, g)
    assert st == 1 and "reserve_space_2 must have the same number of elements as the batches of x, got 3 and 4" in msg
    st, msg = call(dy, x, T(F32, (9,)), m, m, T(F32, (4, 8)), g, g)
    assert st == 1 and "scale must have the same number of elements" in msg
    st, msg = call(dy, x, g, m, m, T(F32, (4, 8)), T(F32, (7,)), g)
    assert st == 1 and "scale_backprop / offset_backprop must have 8 elements" in msg
    # everything valid but no workspace: rejected by the kernel-level check, still no launch
    st, msg = call(dy, x, g, m, m, T(F32, (4, 8), 0x2000), g, g)
    assert st == 1 and "workspace" in msg


def test_fused_instance_norm_validation(L):
    F32, F16 = _capi.ATEXN_F32, _capi.ATEXN_F16

    def call(x, scale, offset, fmt, y, m, r):
        st = L.atexn_fused_instance_norm(ctypes.byref(x), ctypes.byref(scale), ctypes.byref(offset), 1e-3, fmt,
                                         ctypes.byref(y), ctypes.byref(m), ctypes.byref(r), None, 0, None)
        return st, L.atexn_last_error().decode()

    x = T(F16, (2, 8, 8, 32))
    y, st_ = T(F16, (2, 8, 8, 32)), T(F32, (2, 32))
    st, msg = call(T(F16, (2, 8, 32)), T(F32, (32,)), T(F32, (32,)), b"N...C", T(F16, (2, 8, 32)), st_, st_)
    assert st == 1 and "input must be at least 4-dimensional" in msg
    st, msg = call(x, T(F32, (4, 8)), T(F32, (32,)), b"N...C", y, st_, st_)
    assert st == 1 and "scale must be 1-dimensional" in msg
    st, msg = call(x, T(F32, (8,)), T(F32, (32,)), b"N...C", y, st_, st_)
    assert st == 1 and "scale must have the same number of elements as the channels of x, got 8 and 32" in msg
    st, msg = call(x, T(F32, (8,)), T(F32, (8,)), b"NC...", y, T(F32, (2, 9)), st_)
    assert st == 1 and "reserve spaces must have shape [2, 8]" in msg
    st, msg = call(x, T(F32, (32,)), T(F32, (32,)), b"NXYZ", y, st_, st_)
    assert st == 1 and "We only accept" in msg
    e = T(F32, (0, 0, 0, 0, 0), 0)
    z = T(F32, (0,), 0)
    st, msg = call(e, z, z, b"NC...", T(F32, (0, 0, 0, 0, 0), 0), T(F32, (0, 0), 0), T(F32, (0, 0), 0))
    assert st == 0, msg


def test_kernel_level_validation(L):
    assert L.atexn_layer_norm_fwd(9, FAKE, FAKE, FAKE, 4, 8, 1e-3, FAKE, FAKE, FAKE, None, 0, None) == 1
    assert b"bad dtype" in L.atexn_last_error()
    assert L.atexn_layer_norm_fwd(0, FAKE, FAKE, FAKE, -1, 8, 1e-3, FAKE, FAKE, FAKE, None, 0, None) == 1
    assert L.atexn_layer_norm_fwd(0, None, FAKE, FAKE, 4, 8, 1e-3, FAKE, FAKE, FAKE, None, 0, None) == 1
    assert b"NULL pointer" in L.atexn_last_error()
    assert L.atexn_layer_norm_fwd(0, FAKE, FAKE, FAKE, 4, 8, 1e-3, FAKE, FAKE, FAKE, 0x1010, 4096, None) == 1
    assert b"256-byte aligned" in L.atexn_last_error()
    assert L.atexn_layer_norm_bwd(0, FAKE, FAKE, FAKE, FAKE, FAKE, 4, 8, FAKE, FAKE, FAKE, None, 0, None) == 1
    assert L.atexn_layer_norm_bwd(0, FAKE, 0x2000, FAKE, FAKE, FAKE, 4, 8, 0x2000, FAKE, FAKE, 0x4000, 1 << 20, None) == 1
    assert b"dx must not alias x" in L.atexn_last_error()
    assert L.atexn_instance_norm_fwd(0, 5, FAKE, FAKE, FAKE, 1, 2, 3, 1e-3, FAKE, FAKE, FAKE, None, 0, None) == 1
    assert b"bad layout" in L.atexn_last_error()
    # too small a workspace is an argument error, not a launch
    need = L.atexn_layer_norm_bwd_workspace_bytes(1, 8192, 1024)
    assert need > 0
    assert L.atexn_layer_norm_bwd(1, FAKE, 0x2000, FAKE, FAKE, FAKE, 8192, 1024, 0x3000, FAKE, FAKE,
                                  0x4000, need - 256, None) == 1
    assert b"workspace too small" in L.atexn_last_error()
    # the product library has no process-wide settings at all
    assert not hasattr(L, "atexn_set_tuning")
    # the static-scratch backward refuses what does not fit its buffer before it touches a device
    assert L.atexn_layer_norm_bwd_workspace_bytes(1, 2048, 12288) > (8 << 20)
    assert L.atexn_layer_norm_bwd_static(1, FAKE, 0x2000, FAKE, FAKE, FAKE, 2048, 12288, 0x3000, FAKE,
                                         FAKE, None) == 1
    assert b"static buffer" in L.atexn_last_error()


def test_every_planning_parameter_is_settable_in_the_benchmark_build():
    """Each parameter of the planner (struct Tuning in csrc/plan.h) is reachable through the
    benchmark build's atexn_set_tuning under its own name and accepts its default."""
    import os
    import re

    L = _capi.bench_lib()
    assert L.atexn_set_tuning(b"no_such_parameter", 1) == 1
    assert b"unknown tuning parameter" in L.atexn_last_error()

    plan_h = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "atex_amd", "csrc", "plan.h")
    names = re.findall(r"^\s*TuneInt\s+(\w+)\{(\d+)\};", open(plan_h).read(), re.M)
    assert len(names) >= 20
    for name, default in names:
        rc = L.atexn_set_tuning(name.encode(), int(default))
        assert rc == 0, (name, default, L.atexn_last_error())
    # a plan follows its parameter: planes staged on chip need no workspace, planes spread over
    # the workgroups of an XCD need 16 + 4 bytes per chunk, the two-stage kernels 8
    rows = (1, 0, 16, 64, 65536)  # dtype f16, channel-first, N, C, D
    default = L.atexn_instance_norm_fwd_workspace_bytes(*rows)
    assert default == (16 + 4) * 16 * 64 * 2 == _capi.lib().atexn_instance_norm_fwd_workspace_bytes(*rows)
    assert L.atexn_set_tuning(b"plane_single", 0) == 0
    try:
        assert L.atexn_instance_norm_fwd_workspace_bytes(*rows) == 0
        assert L.atexn_set_tuning(b"staged_rows", 0) == 0
        assert L.atexn_instance_norm_fwd_workspace_bytes(*rows) > 0
        # ... and the product library, loaded beside it, is not affected
        assert _capi.lib().atexn_instance_norm_fwd_workspace_bytes(*rows) == default
    finally:
        assert L.atexn_set_tuning(b"staged_rows", 1) == 0
        assert L.atexn_set_tuning(b"plane_single", 1) == 0
    buf = ctypes.create_string_buffer(256)
    assert L.atexn_bench_describe_bwd(0, 1, 0, 8192, 0, 1024, buf, 256) > 0
    assert b"rows_bwd_resident" in buf.value and b"alone=1" in buf.value
    assert L.atexn_bench_describe_bwd(1, 1, 1, 8, 64, 16384, buf, 256) > 0
    assert b"cl_bwd_single" in buf.value and b"alone=0" in buf.value
    assert L.atexn_bench_describe_bwd(1, 1, 1, 2, 32, 2097152, buf, 256) > 0
    assert b"cl_bwd_sums" in buf.value and b"alone=0" in buf.value
    assert L.atexn_bench_describe_bwd(1, 1, 0, 2, 32, 2097152, buf, 256) > 0
    assert b"plane_bwd_single (S=64" in buf.value and b"folded over the batch" in buf.value


def test_workspace_queries_without_gpu(L):
    """Usable on a host without a GPU (they assume 256 CUs) and monotone in the obvious way."""
    assert L.atexn_layer_norm_fwd_workspace_bytes(1, 8192, 1024) == 0       # register-resident rows
    assert L.atexn_layer_norm_fwd_workspace_bytes(1, 4, 10 ** 7) > 0        # split rows
    assert L.atexn_layer_norm_bwd_workspace_bytes(1, 8192, 1024) >= 256 * 2 * 1024 * 4
    assert L.atexn_layer_norm_fwd_workspace_bytes(1, 0, 1024) == 0
    assert L.atexn_layer_norm_fwd_workspace_bytes(5, 8, 8) == 0             # bad dtype
    for layout in (0, 1):
        assert L.atexn_instance_norm_bwd_workspace_bytes(1, layout, 8, 64, 16384) > 0
        assert L.atexn_instance_norm_fwd_workspace_bytes(1, layout, 0, 64, 16384) == 0
    assert L.atexn_instance_norm_fwd_workspace_bytes(1, 1, 8, 64, 16384) % 256 == 0


def test_python_layer_semantics_on_cpu():
    """The wrappers' own checks (reference: nv_norm_ops.py:86-93, :152-158) run before any
    device work; valid calls on host tensors run the library's CPU kernels."""
    import torch

    from atex_amd import nv_norms

    x = torch.zeros(2, 3, 4)
    for axis in ([2, 1], [-1, 1]):  # becomes [2, 1] / [2, 1] after wrapping: unsorted
        layer = nv_norms.LayerNormalization(axis=axis)
        with pytest.raises(ValueError, match="sorted and unique axis"):
            layer(x)
    with pytest.raises(ValueError, match="Duplicate axis"):
        nv_norms.LayerNormalization(axis=[1, 1])(x)
    with pytest.raises(ValueError, match="Invalid axis"):
        nv_norms.LayerNormalization(axis=[5])(x)
    for axis in (2, 0, -2):
        with pytest.raises(ValueError, match="integer axis of 1 or -1"):
            nv_norms.InstanceNormalization(axis=axis)(torch.zeros(2, 3, 4, 5))
    ln = nv_norms.LayerNormalization(axis=[1, -1])   # [1, 2] after wrapping: accepted
    ln.build((2, 3, 4))
    assert tuple(ln.gamma.shape) == (3, 4) and ln.gamma.dtype == torch.float32
    assert [tuple(w.shape) for w in ln.get_weights()] == [(3, 4), (3, 4)]
    assert tuple(ln(x).shape) == (2, 3, 4)
    inn = nv_norms.InstanceNormalization(axis=1)
    inn.build((2, 7, 4, 5))
    assert tuple(inn.gamma.shape) == (7,) and inn.beta.dtype == torch.float32
    assert inn(torch.zeros(2, 7, 4, 5, dtype=torch.float16)).dtype == torch.float16
    assert set(n for n in dir(nv_norms) if not n.startswith("__")) >= {
        "LayerNormalization", "InstanceNormalization", "fused_layer_norm_op", "fused_layer_norm_grad_op",
        "fused_instance_norm_op", "fused_instance_norm_grad_op", "_layer_norm_grad", "_instance_norm_grad"}


def test_header_is_plain_c_and_links_from_c(tmp_path):
    """include/atex_norms.h compiles as C99 and as C++, and a C program linked against the
    library can use the host-side entry points (no Python, no torch, no GPU)."""
    import shutil
    import subprocess

    from atex_amd.nv_norms import _capi

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    inc = os.path.join(root, "include")
    hdr = os.path.join(inc, "atex_norms.h")
    subprocess.run(["gcc", "-std=c99", "-pedantic", "-Wall", "-Werror", "-fsyntax-only", "-x", "c", hdr],
                   check=True)
    subprocess.run(["g++", "-std=c++17", "-Wall", "-Werror", "-fsyntax-only", "-x", "c++", hdr], check=True)
    exe = str(tmp_path / "capi_host_check")
    libdir = os.path.dirname(_capi.LIB_PATH)
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-I", inc,
                    os.path.join(root, "tests", "capi_host_check.c"), "-o", exe,
                    "-L", libdir, "-latex_norms_hip", f"-Wl,-rpath,{libdir}"], check=True)
    out = subprocess.run([exe], capture_output=True, text=True, timeout=60)
    assert out.returncode == 0, out.stderr + out.stdout
    assert "capi host check ok" in out.stdout


# ------------------------------------------------------------------ property tests
def _axes_model(dims, axis):
    """Python restatement of GetBatchAndFeatureSizes (cc/ops/norm_ops.cc:18-52): wrap negative
    axes, reject out-of-range ones, sort, drop duplicates, require the set to be packed up to
    the last dim.  Returns (N, D) or an error word."""
    rank = len(dims)
    wrapped = []
    for a in axis:
        w = a + rank if a < 0 else a
        if w < 0 or w >= rank:
            return "invalid"
        wrapped.append(w)
    uniq = sorted(set(wrapped))
    if uniq[0] != rank - len(uniq):
        return "packed"
    n = d = 1
    for i, v in enumerate(dims):
        if i >= uniq[0]:
            d *= v
        else:
            n *= v
    return n, d


def test_axis_resolution_property(L):
    from hypothesis import given, settings
    from hypothesis import strategies as st

    @settings(max_examples=400, deadline=None)
    @given(st.lists(st.integers(0, 9), min_size=1, max_size=6).flatmap(
        lambda dims: st.tuples(st.just(dims),
                               st.lists(st.integers(-len(dims) - 2, len(dims) + 1), min_size=1, max_size=7))))
    def check(case):
        dims, axis = case
        want = _axes_model(dims, axis)
        st_, n, d, msg = resolve_axes(L, dims, axis)
        if want == "invalid":
            assert st_ == 1 and "axis contains invalid value" in msg
        elif want == "packed":
            assert st_ == 1 and "axis is not packed from last dim." in msg
        else:
            assert st_ == 0 and (n, d) == want

    check()


def test_data_format_property(L):
    """fused_instance_norm_op.cc:25-34: accepted iff len > 2, [0] == 'N' and ([1] == 'C' or
    [-1] == 'C'); a 'C' in position 1 wins."""
    from hypothesis import given, settings
    from hypothesis import strategies as st

    @settings(max_examples=400, deadline=None)
    @given(st.text(alphabet="NCHWD.x", min_size=0, max_size=7), st.lists(st.integers(0, 6), min_size=4, max_size=6))
    def check(fmt, dims):
        ok = len(fmt) > 2 and fmt[0] == "N" and (fmt[1] == "C" or fmt[-1] == "C")
        st_, layout, n, c, d, msg = resolve_format(L, dims, fmt.encode())
        if not ok:
            assert st_ == 1 and "We only accept" in msg
            return
        cf = fmt[1] == "C"
        spatial = dims[2:] if cf else dims[1:-1]
        prod = 1
        for v in spatial:
            prod *= v
        assert st_ == 0 and layout == (0 if cf else 1)
        assert (n, c, d) == (dims[0], dims[1] if cf else dims[-1], prod)

    check()
