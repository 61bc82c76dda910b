"""The library's host (CPU) kernels, the counterpart of the reference's registered CPU
kernels (cc/kernels/fused_layer_norm_op.cc:27-223, :465-478; fused_instance_norm_op.cc:39-284,
:541-554): kernel-level atexn_*_cpu entry points against the committed golden fixtures and
the oracle's float64 flavour, the op level on host tensors, the layers with autograd, empty
inputs, and independence of the result from the number of host threads.  No GPU needed.
"""
import ctypes
import glob
import hashlib
import os
import subprocess
import sys

import numpy as np
import pytest

from oracle import oracle as O
from tests import util
from tests.util import TOL, assert_close

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "*.npz")))
EPS = 1e-3


class CpuCapi:
    """Kernel-level CPU entry points on numpy arrays in storage representation."""

    def __init__(self):
        from atex_amd.nv_norms import _capi

        self.capi = _capi
        self.L = _capi.lib()

    @staticmethod
    def _p(a):
        return a.ctypes.data_as(ctypes.c_void_p) if a.size else None

    def ln_fwd(self, x, gamma, beta, eps, dtype):
        N, D = x.shape
        y = np.empty_like(x)
        mean, rstd = np.empty(N, np.float32), np.empty(N, np.float32)
        self.capi.check(self.L.atexn_layer_norm_fwd_cpu(O.DTYPE_CODE[dtype], self._p(x), self._p(gamma), self._p(beta),
                                                       N, D, eps, self._p(y), self._p(mean), self._p(rstd)))
        return y, mean, rstd

    def ln_bwd(self, dy, x, gamma, mean, rstd, dtype):
        N, D = x.shape
        dx = np.empty_like(x)
        dg, db = np.full(D, np.nan, np.float32), np.full(D, np.nan, np.float32)
        self.capi.check(self.L.atexn_layer_norm_bwd_cpu(O.DTYPE_CODE[dtype], self._p(dy), self._p(x), self._p(gamma),
                                                       self._p(mean), self._p(rstd), N, D, self._p(dx),
                                                       self._p(dg), self._p(db)))
        return dx, dg, db

    def in_fwd(self, x, gamma, beta, eps, dtype, cf):
        N, C, D = (x.shape[0], x.shape[1], x.shape[2]) if cf else (x.shape[0], x.shape[2], x.shape[1])
        y = np.empty_like(x)
        mean, rstd = np.empty((N, C), np.float32), np.empty((N, C), np.float32)
        self.capi.check(self.L.atexn_instance_norm_fwd_cpu(O.DTYPE_CODE[dtype], 0 if cf else 1, self._p(x),
                                                          self._p(gamma), self._p(beta), N, C, D, eps,
                                                          self._p(y), self._p(mean), self._p(rstd)))
        return y, mean, rstd

    def in_bwd(self, dy, x, gamma, mean, rstd, dtype, cf):
        N, C, D = (x.shape[0], x.shape[1], x.shape[2]) if cf else (x.shape[0], x.shape[2], x.shape[1])
        dx = np.empty_like(x)
        dg, db = np.full(C, np.nan, np.float32), np.full(C, np.nan, np.float32)
        self.capi.check(self.L.atexn_instance_norm_bwd_cpu(O.DTYPE_CODE[dtype], 0 if cf else 1, self._p(dy),
                                                          self._p(x), self._p(gamma), self._p(mean),
                                                          self._p(rstd), N, C, D, self._p(dx), self._p(dg),
                                                          self._p(db)))
        return dx, dg, db


@pytest.fixture(scope="module")
def cpu():
    return CpuCapi()


def _vals(a, dtype):
    return O.from_storage(a, dtype)


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p)[:-4] for p in GOLDEN])
def test_cpu_kernels_match_golden(cpu, path):
    g = np.load(path)
    dtype, eps, kind = str(g["dtype"]), float(g["eps"]), str(g["kind"])
    tol = TOL[dtype]
    x, dy = np.ascontiguousarray(g["x"]), np.ascontiguousarray(g["dy"])
    gamma, beta = g["gamma"], g["beta"]
    mean32, rstd32 = g["mean"].astype(np.float32), g["inv_std"].astype(np.float32)
    if kind == "ln":
        y, m, r = cpu.ln_fwd(x, gamma, beta, eps, dtype)
        dx, dg, db = cpu.ln_bwd(dy, x, gamma, mean32, rstd32, dtype)
    else:
        cf = bool(g["channel_first"])
        y, m, r = cpu.in_fwd(x, gamma, beta, eps, dtype, cf)
        dx, dg, db = cpu.in_bwd(dy, x, gamma, mean32, rstd32, dtype, cf)
    assert_close(m, g["mean"], tol["stat"], "mean")
    assert_close(r, g["inv_std"], tol["stat"], "inv_std")
    assert_close(_vals(y, dtype), g["y"], tol["y"], "y")
    scale = util.dx_scale(g["dy"], np.sqrt(np.mean(gamma.astype(np.float64) ** 2)), g["inv_std"], dtype)
    assert_close(_vals(dx, dtype), g["dx"], tol["dx"], "dx", scale=scale)
    assert_close(dg, g["dgamma"], tol["dw"], "dgamma")
    assert_close(db, g["dbeta"], tol["dw"], "dbeta")


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("N,D", [(32, 1024), (300, 1000), (3, 40001), (5000, 10), (1, 1), (7, 70000), (2, 1 << 18)])
def test_layer_norm_cpu_vs_oracle(cpu, coracle, N, D, dtype):
    x, gamma, beta, dy = util.ln_inputs("row_mean", N, D, dtype, 50)
    y_ref, m_ref, r_ref = coracle.ln_fwd(x, gamma, beta, EPS, dtype)
    y, m, r = cpu.ln_fwd(x, gamma, beta, EPS, dtype)
    tol = TOL[dtype]
    assert_close(m, m_ref, 1e-5, "mean")          # statistics are float32 whatever the storage type
    assert_close(r, r_ref, 1e-5, "inv_std")
    assert_close(_vals(y, dtype), y_ref, tol["y"], "y")
    m32, r32 = m_ref.astype(np.float32), r_ref.astype(np.float32)
    dx_ref, dg_ref, db_ref = coracle.ln_bwd(dy, x, gamma, m32.astype(np.float64), r32.astype(np.float64), dtype)
    dx, dg, db = cpu.ln_bwd(dy, x, gamma, m32, r32, dtype)
    assert_close(_vals(dx, dtype), dx_ref, tol["dx"], "dx",
                 scale=util.dx_scale(dy, np.sqrt(np.mean(gamma.astype(np.float64) ** 2)), r32, dtype))
    assert_close(dg, dg_ref, 1e-5, "dgamma")      # sums carried in double
    assert_close(db, db_ref, 1e-5, "dbeta")


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("channel_first", [False, True])
@pytest.mark.parametrize("N,C,S", [(2, 32, 1024), (3, 5, 777), (1, 64, 16384), (4, 3, 1), (2, 100, 50), (600, 8, 20)])
def test_instance_norm_cpu_vs_oracle(cpu, coracle, N, C, S, channel_first, dtype):
    x, gamma, beta, dy = util.in_inputs(N, C, S, dtype, channel_first, 51)
    y_ref, m_ref, r_ref = coracle.in_fwd(x, gamma, beta, EPS, dtype, channel_first)
    y, m, r = cpu.in_fwd(x, gamma, beta, EPS, dtype, channel_first)
    tol = TOL[dtype]
    assert_close(m, m_ref, 1e-5, "mean")
    assert_close(r, r_ref, 1e-5, "inv_std")
    assert_close(_vals(y, dtype), y_ref, tol["y"], "y")
    m32, r32 = m_ref.astype(np.float32), r_ref.astype(np.float32)
    dx_ref, dg_ref, db_ref = coracle.in_bwd(dy, x, gamma, m32.astype(np.float64), r32.astype(np.float64), dtype,
                                            channel_first)
    dx, dg, db = cpu.in_bwd(dy, x, gamma, m32, r32, dtype, channel_first)
    assert_close(_vals(dx, dtype), dx_ref, tol["dx"], "dx",
                 scale=util.dx_scale(dy, np.sqrt(np.mean(gamma.astype(np.float64) ** 2)), r32, dtype))
    assert_close(dg, dg_ref, 1e-5, "dgamma")
    assert_close(db, db_ref, 1e-5, "dbeta")


def test_storage_conversions_every_pattern(cpu):
    """The CPU kernels' own half / bfloat16 conversions, through the kernels: a row [v, -v] has
    mean 0 and, with eps = 0, inv_std = 1 / |v|, so y = (+-1) * gamma + beta; gamma = |v| gives
    back v after one load and one store.  Run for every positive finite 16-bit pattern whose
    square stays inside the float32 range (all of half, 2^-60 .. 2^60 of bfloat16), as the
    channels (= rows with their own gamma) of one channel-first instance."""
    for dtype, to_f32 in (("f16", lambda b: b.view(np.float16).astype(np.float32)),
                          ("bf16", O.bf16_bits_to_f32)):
        bits = np.arange(0, 0x8000, dtype=np.uint16)
        vals = to_f32(bits)
        keep = np.isfinite(vals) & (vals > 2.0 ** -60) & (vals < 2.0 ** 60)
        bits, vals = bits[keep], vals[keep]
        x = np.stack([bits, bits | 0x8000], axis=1)                 # rows [v, -v]
        x = x.view(np.float16) if dtype == "f16" else x
        C = x.shape[0]
        xi = np.ascontiguousarray(x.reshape(1, C, 2))
        y, m, r = cpu.in_fwd(xi, vals.astype(np.float32), np.zeros(C, np.float32), 0.0, dtype, True)
        got = y.reshape(C, 2).view(np.uint16).astype(np.int32)
        want = x.view(np.uint16).astype(np.int32)
        # (1 / |v|) * |v| may be one float32 ulp off 1: invisible after rounding to 16 bits
        # except next to a rounding boundary
        diff = np.abs(got - want)
        assert diff.max() <= 1, (dtype, int(diff.max()))
        assert (diff > 0).mean() < 1e-3, (dtype, float((diff > 0).mean()))
        assert np.all(m == 0.0)


def test_empty_inputs_zero_fill(cpu):
    dg = np.full(16, 7.0, np.float32)
    db = np.full(16, 7.0, np.float32)
    g = np.ones(16, np.float32)
    L = cpu.L
    st = L.atexn_layer_norm_bwd_cpu(0, None, None, g.ctypes.data_as(ctypes.c_void_p), None, None, 0, 16, None,
                                    dg.ctypes.data_as(ctypes.c_void_p), db.ctypes.data_as(ctypes.c_void_p))
    assert st == 0 and not dg.any() and not db.any()
    dg[:] = 7.0
    db[:] = 7.0
    for layout in (0, 1):
        st = L.atexn_instance_norm_bwd_cpu(0, layout, None, None, g.ctypes.data_as(ctypes.c_void_p), None, None,
                                           0, 16, 5, None, dg.ctypes.data_as(ctypes.c_void_p),
                                           db.ctypes.data_as(ctypes.c_void_p))
        assert st == 0 and not dg.any() and not db.any()
    assert L.atexn_layer_norm_fwd_cpu(0, None, None, None, 0, 0, 1e-3, None, None, None) == 0
    assert L.atexn_layer_norm_fwd_cpu(7, None, None, None, 1, 1, 1e-3, None, None, None) == 1
    assert L.atexn_layer_norm_fwd_cpu(0, None, None, None, 1, 1, 1e-3, None, None, None) == 1


_THREAD_PROBE = r"""
import hashlib, sys
import numpy as np
sys.path.insert(0, %(root)r)
from tests import util
from tests.test_cpu_kernels import CpuCapi
cpu = CpuCapi()
h = hashlib.sha256()
x, gamma, beta, dy = util.ln_inputs("row_mean", 700, 1024, "f16", 52)
y, m, r = cpu.ln_fwd(x, gamma, beta, 1e-3, "f16")
dx, dg, db = cpu.ln_bwd(dy, x, gamma, m, r, "f16")
for a in (y, m, r, dx, dg, db): h.update(a.tobytes())
x, gamma, beta, dy = util.ln_inputs("plain", 40, 8192, "f32", 53)
y, m, r = cpu.ln_fwd(x, gamma, beta, 1e-3, "f32")
dx, dg, db = cpu.ln_bwd(dy, x, gamma, m, r, "f32")
for a in (y, m, r, dx, dg, db): h.update(a.tobytes())
for cf in (False, True):
    x, gamma, beta, dy = util.in_inputs(3, 16, 5000, "f16", cf, 54)
    y, m, r = cpu.in_fwd(x, gamma, beta, 1e-3, "f16", cf)
    dx, dg, db = cpu.in_bwd(dy, x, gamma, m, r, "f16", cf)
    for a in (y, m, r, dx, dg, db): h.update(a.tobytes())
print(h.hexdigest())
"""


def test_results_do_not_depend_on_thread_count():
    digests = set()
    for threads in ("1", "3", "8"):
        env = dict(os.environ, ATEXN_CPU_THREADS=threads)
        out = subprocess.run([sys.executable, "-c", _THREAD_PROBE % {"root": ROOT}], env=env, capture_output=True,
                             text=True, check=True).stdout.strip()
        digests.add(out)
    assert len(digests) == 1, digests


def test_op_level_and_layers_on_host_tensors():
    """Host tensors through the op level (device field of the descriptors) and through the
    layers with autograd, against torch's own float32 layer_norm / group_norm."""
    import torch

    from atex_amd import nv_norms

    torch.manual_seed(5)
    x = torch.randn(6, 5, 32, requires_grad=True)
    ln = nv_norms.LayerNormalization(axis=[1, 2], epsilon=EPS)
    y = ln(x)
    with torch.no_grad():
        ln.gamma.copy_(torch.rand(5, 32) + 0.5)
        ln.beta.copy_(torch.randn(5, 32) * 0.1)
    y = ln(x)
    (y * torch.arange(y.numel(), dtype=torch.float32).reshape(y.shape) / y.numel()).sum().backward()
    xr = x.detach().clone().requires_grad_(True)
    g, b = ln.gamma.detach().clone().requires_grad_(True), ln.beta.detach().clone().requires_grad_(True)
    yr = torch.nn.functional.layer_norm(xr, (5, 32), g, b, EPS)
    (yr * torch.arange(y.numel(), dtype=torch.float32).reshape(y.shape) / y.numel()).sum().backward()
    assert torch.allclose(y, yr, rtol=1e-5, atol=1e-6)
    assert torch.allclose(x.grad, xr.grad, rtol=1e-4, atol=1e-6)
    assert torch.allclose(ln.gamma.grad, g.grad, rtol=1e-4, atol=1e-6)
    assert torch.allclose(ln.beta.grad, b.grad, rtol=1e-4, atol=1e-6)

    for axis, fmt in ((1, "cf"), (-1, "cl")):
        C = 7
        shape = (2, C, 6, 5) if fmt == "cf" else (2, 6, 5, C)
        xi = torch.randn(shape, requires_grad=True)
        inn = nv_norms.InstanceNormalization(axis=axis, epsilon=EPS)
        yi = inn(xi)
        yi.square().sum().backward()
        xc = xi.detach().clone().requires_grad_(True)
        xc_cf = xc if fmt == "cf" else xc.permute(0, 3, 1, 2)
        ref = torch.nn.functional.group_norm(xc_cf, C, inn.gamma.detach(), inn.beta.detach(), EPS)
        ref = ref if fmt == "cf" else ref.permute(0, 2, 3, 1)
        ref.square().sum().backward()
        assert torch.allclose(yi, ref, rtol=1e-5, atol=1e-6)
        assert torch.allclose(xi.grad, xc.grad, rtol=1e-4, atol=1e-5)

    # the op level refuses tensors on different devices before anything runs
    from atex_amd.nv_norms import _capi

    L = _capi.lib()
    a = np.zeros((2, 4), np.float32)
    t_cpu = _capi.make_tensor(0, (2, 4), a.ctypes.data, _capi.ATEXN_DEVICE_CPU)
    t_gpu = _capi.make_tensor(0, (2, 4), a.ctypes.data, _capi.ATEXN_DEVICE_GPU)
    w = _capi.make_tensor(0, (4,), a.ctypes.data, _capi.ATEXN_DEVICE_CPU)
    s = _capi.make_tensor(0, (2,), a.ctypes.data, _capi.ATEXN_DEVICE_CPU)
    ax = (ctypes.c_int * 1)(-1)
    st = L.atexn_fused_layer_norm(ctypes.byref(t_cpu), ctypes.byref(w), ctypes.byref(w), 1e-3, ax, 1,
                                  ctypes.byref(t_gpu), ctypes.byref(s), ctypes.byref(s), None, 0, None)
    assert st == 1 and b"same device" in L.atexn_last_error()
    assert L.atexn_fused_layer_norm_workspace_bytes(ctypes.byref(t_cpu), ax, 1) == 0


def test_cpu_kernels_random_shapes(cpu):
    """Seeded random shapes (rows of 1 .. 5000 elements, 1 .. 40 rows / instances, both layouts,
    every dtype) against the numpy float64 closed forms."""
    rng = np.random.Generator(np.random.PCG64(77))
    for case in range(120):
        dtype = ("f32", "f16", "bf16")[case % 3]
        tol = TOL[dtype]
        if case % 2 == 0:
            N, D = int(rng.integers(1, 40)), int(rng.integers(1, 5000))
            x, gamma, beta, dy = util.ln_inputs("row_mean", N, D, dtype, 1000 + case)
            xv, dyv = O.from_storage(x, dtype), O.from_storage(dy, dtype)
            y_ref, m_ref, r_ref = O.ln_fwd_np(xv, gamma, beta, EPS)
            y, m, r = cpu.ln_fwd(x, gamma, beta, EPS, dtype)
            m32, r32 = m_ref.astype(np.float32), r_ref.astype(np.float32)
            dx_ref, dg_ref, db_ref = O.ln_bwd_np(dyv, xv, gamma, m32, r32)
            dx, dg, db = cpu.ln_bwd(dy, x, gamma, m32, r32, dtype)
        else:
            N, C, S = int(rng.integers(1, 6)), int(rng.integers(1, 70)), int(rng.integers(1, 900))
            cf = bool(rng.integers(0, 2))
            x, gamma, beta, dy = util.in_inputs(N, C, S, dtype, cf, 1000 + case)
            xv, dyv = O.from_storage(x, dtype), O.from_storage(dy, dtype)
            y_ref, m_ref, r_ref = O.in_fwd_np(xv, gamma, beta, EPS, cf)
            y, m, r = cpu.in_fwd(x, gamma, beta, EPS, dtype, cf)
            m32, r32 = m_ref.astype(np.float32), r_ref.astype(np.float32)
            dx_ref, dg_ref, db_ref = O.in_bwd_np(dyv, xv, gamma, m32, r32, cf)
            dx, dg, db = cpu.in_bwd(dy, x, gamma, m32, r32, dtype, cf)
        what = f"case {case} {dtype} x{x.shape}"
        assert_close(m, m_ref, 1e-5, what + " mean")
        assert_close(r, r_ref, 1e-5, what + " inv_std")
        assert_close(_vals(y, dtype), y_ref, tol["y"], what + " y")
        scale = util.dx_scale(dy, np.sqrt(np.mean(gamma.astype(np.float64) ** 2)), r32, dtype)
        assert_close(_vals(dx, dtype), dx_ref, tol["dx"], what + " dx", scale=scale)
        assert_close(dg, dg_ref, 1e-5, what + " dgamma")
        assert_close(db, db_ref, 1e-5, what + " dbeta")
