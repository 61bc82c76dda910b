"""Pins the CPU oracle (oracle/norms_oracle.c and the numpy restatement) WITHOUT using it to
check itself:

* golden fixtures produced by torch's CPU float64 native_layer_norm / group_norm + autograd
  (tests/golden/make_golden.py) -- an independent implementation of the same mathematics;
* the numpy closed forms of the reference's own tests, typed here following
  tests/fused_layer_norm_test.py:20-62 and tests/fused_instance_norm_test.py:21-65;
* what the mathematics fixes: central finite differences of a scalar loss on tiny inputs,
  row invariants of dx, the constant-row and D = 1 special cases, shift invariance, the
  saved-statistic convention inv_std^2 = 1 / (var + eps) (fused_layer_norm_test.py:84),
  and the layout equivalence of the two InstanceNorm formats;
* the fp16 / bf16 conversions against numpy / torch for every 16-bit pattern.

NOT pinned (no TensorFlow here): the last-ulp fp16 rounding of tf.keras / tensorflow_addons.
"""
import glob
import os

import numpy as np
import pytest
import torch

from oracle import oracle as O

GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "*.npz")))


def _close(a, b, rtol, what):
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    scale = max(float(np.sqrt(np.mean(b * b))), 1e-30)
    err = np.abs(a - b)
    assert np.all(err <= rtol * np.abs(b) + rtol * scale), f"{what}: max err {err.max():.3e}, scale {scale:.3e}"


def _x64(g, key):
    return O.from_storage(g[key], str(g["dtype"]))


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p)[:-4] for p in GOLDEN])
@pytest.mark.parametrize("impl", ["c_f64", "numpy"])
def test_oracle_matches_golden(coracle, path, impl):
    g = np.load(path)
    dtype, eps = str(g["dtype"]), float(g["eps"])
    # y / dx are stored as float32 in the fixtures
    tol_big = 2e-7
    if str(g["kind"]) == "ln":
        if impl == "c_f64":
            y, m, r = coracle.ln_fwd(g["x"], g["gamma"], g["beta"], eps, dtype)
            dx, dg, db = coracle.ln_bwd(g["dy"], g["x"], g["gamma"], g["mean"], g["inv_std"], dtype)
        else:
            y, m, r = O.ln_fwd_np(_x64(g, "x"), g["gamma"], g["beta"], eps)
            dx, dg, db = O.ln_bwd_np(_x64(g, "dy"), _x64(g, "x"), g["gamma"], g["mean"], g["inv_std"])
    else:
        cf = bool(g["channel_first"])
        if impl == "c_f64":
            y, m, r = coracle.in_fwd(g["x"], g["gamma"], g["beta"], eps, dtype, cf)
            dx, dg, db = coracle.in_bwd(g["dy"], g["x"], g["gamma"], g["mean"], g["inv_std"], dtype, cf)
        else:
            y, m, r = O.in_fwd_np(_x64(g, "x"), g["gamma"], g["beta"], eps, cf)
            dx, dg, db = O.in_bwd_np(_x64(g, "dy"), _x64(g, "x"), g["gamma"], g["mean"], g["inv_std"], cf)
    _close(m, g["mean"], 1e-11, "mean")
    _close(r, g["inv_std"], 1e-11, "inv_std")
    _close(y, g["y"], tol_big, "y")
    _close(dx, g["dx"], tol_big, "dx")
    _close(dg, g["dgamma"], 1e-10, "dgamma")
    _close(db, g["dbeta"], 1e-10, "dbeta")


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p)[:-4] for p in GOLDEN])
def test_float_flavour_matches_golden(coracle, path):
    """The float flavour (reference arithmetic, also the timed CPU baseline) stays within
    the op's tolerance of the float64 truth."""
    g = np.load(path)
    dtype, eps = str(g["dtype"]), float(g["eps"])
    tol = 2e-5 if dtype == "f32" else 1e-2
    if str(g["kind"]) == "ln":
        y, m, r = coracle.ln_fwd(g["x"], g["gamma"], g["beta"], eps, dtype, f64=False)
        dx, dg, db = coracle.ln_bwd(g["dy"], g["x"], g["gamma"], g["mean"], g["inv_std"], dtype, f64=False)
    else:
        cf = bool(g["channel_first"])
        y, m, r = coracle.in_fwd(g["x"], g["gamma"], g["beta"], eps, dtype, cf, f64=False)
        dx, dg, db = coracle.in_bwd(g["dy"], g["x"], g["gamma"], g["mean"], g["inv_std"], dtype, cf, f64=False)
    _close(m, g["mean"], 1e-4, "mean")
    _close(r, g["inv_std"], 1e-4, "inv_std")
    _close(O.from_storage(y, dtype), g["y"], tol, "y")
    _close(O.from_storage(dx, dtype), g["dx"], tol, "dx")
    _close(dg, g["dgamma"], 1e-3, "dgamma")
    _close(db, g["dbeta"], 1e-3, "dbeta")


# ----------------------------------------------------- the reference tests' closed forms
def layer_norm_grad_reference_test_form(x, dy, gamma, mean, istd):
    """fused_layer_norm_test.py:20-62, on [N, D] float64 arrays."""
    N, D = x.shape
    mean = mean[:, None]
    istd = istd[:, None]
    x_mean = x - mean
    dgamma = np.sum(dy * x_mean * istd, axis=0)
    dbeta = np.sum(dy, axis=0)
    dl_di = dy * gamma * istd
    dl_dvar = np.sum(dy * gamma * x_mean * (-0.5) * (istd ** 3), axis=1, keepdims=True)
    dvar_dx = 2.0 * x_mean / D
    dl_dmean = np.sum(-1.0 * dy * gamma * istd, axis=1, keepdims=True)
    dx = dl_di + dl_dvar * dvar_dx + dl_dmean * (1.0 / D)
    return dgamma, dbeta, dx


def instance_norm_grad_reference_test_form(x, dy, gamma, mean, istd, channel_first):
    """fused_instance_norm_test.py:21-65, on [N,C,D] / [N,D,C] float64 arrays."""
    d_axis = (2,) if channel_first else (1,)
    nd_axis = (0,) + d_axis
    D = x.shape[d_axis[0]]
    ex = -1 if channel_first else 1
    istd = np.expand_dims(istd, ex)
    mean = np.expand_dims(mean, ex)
    gamma = np.expand_dims(np.expand_dims(gamma, -1 if channel_first else 0), 0)
    x_mean = x - mean
    dgamma = np.sum(dy * x_mean * istd, axis=nd_axis)
    dbeta = np.sum(dy, axis=nd_axis)
    dl_di = dy * gamma * istd
    dl_dvar = np.sum(dy * gamma * x_mean * (-0.5) * (istd ** 3), axis=d_axis, keepdims=True)
    dl_dmean = np.sum(-1.0 * dy * gamma * istd, axis=d_axis, keepdims=True)
    dx = dl_di + dl_dvar * (2.0 * x_mean / D) + dl_dmean / D
    return dgamma, dbeta, dx


def test_against_reference_test_closed_forms(coracle):
    rng = np.random.default_rng(11)
    x = rng.normal(0, 10, size=(6, 50)).astype(np.float32)
    dy = rng.normal(size=(6, 50)).astype(np.float32)
    gamma = rng.normal(size=50).astype(np.float32)
    mean = x.astype(np.float64).mean(axis=1)
    istd = 1.0 / np.sqrt(x.astype(np.float64).var(axis=1) + 1e-3)
    dg_r, db_r, dx_r = layer_norm_grad_reference_test_form(x.astype(np.float64), dy.astype(np.float64),
                                                          gamma.astype(np.float64), mean, istd)
    dx, dg, db = coracle.ln_bwd(dy, x, gamma, mean, istd, "f32")
    _close(dx, dx_r, 1e-11, "dx")
    _close(dg, dg_r, 1e-11, "dgamma")
    _close(db, db_r, 1e-11, "dbeta")
    for cf in (True, False):
        shape = (2, 3, 40) if cf else (2, 40, 3)
        x = rng.normal(0, 10, size=shape).astype(np.float32)
        dy = rng.normal(size=shape).astype(np.float32)
        gamma = rng.normal(size=3).astype(np.float32)
        ax = 2 if cf else 1
        mean = x.astype(np.float64).mean(axis=ax)
        istd = 1.0 / np.sqrt(x.astype(np.float64).var(axis=ax) + 1e-3)
        dg_r, db_r, dx_r = instance_norm_grad_reference_test_form(
            x.astype(np.float64), dy.astype(np.float64), gamma.astype(np.float64), mean, istd, cf)
        dx, dg, db = coracle.in_bwd(dy, x, gamma, mean, istd, "f32", cf)
        _close(dx, dx_r, 1e-11, "dx")
        _close(dg, dg_r, 1e-11, "dgamma")
        _close(db, db_r, 1e-11, "dbeta")


# ------------------------------------------------------------ what the mathematics fixes
def test_finite_differences_layer_norm(coracle):
    """d/dtheta of L = sum(w * LN(x)) by central differences in float64 (brute force, tiny)."""
    rng = np.random.default_rng(5)
    N, D, eps, h = 3, 7, 1e-3, 1e-6
    x = rng.normal(size=(N, D))
    gamma = rng.uniform(0.5, 1.5, size=D)
    beta = rng.normal(size=D)
    w = rng.normal(size=(N, D))

    def loss(x_, g_, b_):
        m = x_.mean(axis=1, keepdims=True)
        v = ((x_ - m) ** 2).mean(axis=1, keepdims=True)
        return float(np.sum(w * ((x_ - m) / np.sqrt(v + eps) * g_ + b_)))

    def num_grad(arr, which):
        g = np.zeros_like(arr)
        it = np.nditer(arr, flags=["multi_index"])
        for _ in it:
            i = it.multi_index
            ap, am = arr.copy(), arr.copy()
            ap[i] += h
            am[i] -= h
            args_p = [x, gamma, beta]
            args_m = [x, gamma, beta]
            args_p[which], args_m[which] = ap, am
            g[i] = (loss(*args_p) - loss(*args_m)) / (2 * h)
        return g

    x32 = x.astype(np.float32)
    x = x32.astype(np.float64)  # the oracle sees float32 storage
    g32, b32 = gamma.astype(np.float32), beta.astype(np.float32)
    gamma, beta = g32.astype(np.float64), b32.astype(np.float64)
    w32 = w.astype(np.float32)
    w = w32.astype(np.float64)
    _, mean, rstd = coracle.ln_fwd(x32, g32, b32, eps, "f32")
    dx, dg, db = coracle.ln_bwd(w32, x32, g32, mean, rstd, "f32")
    _close(dx, num_grad(x, 0), 1e-6, "dx")
    _close(dg, num_grad(gamma, 1), 1e-6, "dgamma")
    _close(db, num_grad(beta, 2), 1e-6, "dbeta")


def test_finite_differences_instance_norm(coracle):
    rng = np.random.default_rng(6)
    N, C, D, eps, h = 2, 3, 5, 1e-3, 1e-6
    for cf in (True, False):
        shape = (N, C, D) if cf else (N, D, C)
        ax = 2 if cf else 1
        x = rng.normal(size=shape).astype(np.float32).astype(np.float64)
        gamma = rng.uniform(0.5, 1.5, size=C).astype(np.float32).astype(np.float64)
        beta = rng.normal(size=C).astype(np.float32).astype(np.float64)
        w = rng.normal(size=shape).astype(np.float32).astype(np.float64)
        bshape = (1, C, 1) if cf else (1, 1, C)

        def loss(x_, g_, b_):
            m = x_.mean(axis=ax, keepdims=True)
            v = ((x_ - m) ** 2).mean(axis=ax, keepdims=True)
            return float(np.sum(w * ((x_ - m) / np.sqrt(v + eps) * g_.reshape(bshape) + b_.reshape(bshape))))

        def num_grad(arr, which):
            g = np.zeros_like(arr)
            it = np.nditer(arr, flags=["multi_index"])
            for _ in it:
                i = it.multi_index
                ap, am = arr.copy(), arr.copy()
                ap[i] += h
                am[i] -= h
                ap_args, am_args = [x, gamma, beta], [x, gamma, beta]
                ap_args[which], am_args[which] = ap, am
                g[i] = (loss(*ap_args) - loss(*am_args)) / (2 * h)
            return g

        f32 = lambda a: a.astype(np.float32)
        _, mean, rstd = coracle.in_fwd(f32(x), f32(gamma), f32(beta), eps, "f32", cf)
        dx, dg, db = coracle.in_bwd(f32(w), f32(x), f32(gamma), mean, rstd, "f32", cf)
        _close(dx, num_grad(x, 0), 1e-6, "dx")
        _close(dg, num_grad(gamma, 1), 1e-6, "dgamma")
        _close(db, num_grad(beta, 2), 1e-6, "dbeta")


def test_invariants_and_special_cases(coracle):
    rng = np.random.default_rng(7)
    eps = 1e-3
    x = rng.normal(3.0, 2.0, size=(9, 33)).astype(np.float32)
    gamma = rng.uniform(0.5, 1.5, size=33).astype(np.float32)
    beta = rng.normal(size=33).astype(np.float32)
    dy = rng.normal(size=(9, 33)).astype(np.float32)
    y, mean, rstd = coracle.ln_fwd(x, gamma, beta, eps, "f32")
    xd = x.astype(np.float64)
    # saved statistics: biased variance, inverse STD (fused_layer_norm_test.py:84)
    _close(mean, xd.mean(axis=1), 1e-12, "mean")
    _close(rstd ** 2, 1.0 / (xd.var(axis=1) + eps), 1e-12, "inv_std^2")
    # normalised rows: mean 0, variance var / (var + eps)
    z = (y - beta.astype(np.float64)) / gamma.astype(np.float64)
    assert np.abs(z.mean(axis=1)).max() < 1e-12
    _close(z.var(axis=1), xd.var(axis=1) / (xd.var(axis=1) + eps), 1e-10, "var(z)")
    # shift invariance (exact data: shift by a power of two)
    y2, mean2, rstd2 = coracle.ln_fwd(x + np.float32(64.0), gamma, beta, eps, "f32")
    _close(y2, y, 1e-5, "shifted y")  # the shift itself rounds x in float32
    # dx row invariants: sum_j dx = 0, sum_j dx * (x - mean) = eps * r^3 * s2
    dx, dg, db = coracle.ln_bwd(dy, x, gamma, mean, rstd, "f32")
    assert np.abs(dx.sum(axis=1)).max() < 1e-12
    g = dy.astype(np.float64) * gamma.astype(np.float64)
    s2 = (g * (xd - mean[:, None])).sum(axis=1)
    _close((dx * (xd - mean[:, None])).sum(axis=1), eps * rstd ** 3 * s2, 1e-9, "sum dx (x - mean)")
    _close(db, dy.astype(np.float64).sum(axis=0), 1e-12, "dbeta")
    # constant rows: y = beta, inv_std = eps^-1/2; D = 1 likewise
    xc = np.full((4, 16), 2.5, np.float32)
    yc, mc, rc = coracle.ln_fwd(xc, gamma[:16], beta[:16], eps, "f32")
    _close(yc, np.broadcast_to(beta[:16].astype(np.float64), (4, 16)), 1e-12, "constant-row y")
    _close(rc, np.full(4, eps ** -0.5), 1e-12, "constant-row inv_std")
    y1, m1, r1 = coracle.ln_fwd(x[:, :1].copy(), gamma[:1], beta[:1], eps, "f32")
    _close(y1, np.broadcast_to(beta[:1].astype(np.float64), (9, 1)), 1e-12, "D=1 y")
    _close(m1, xd[:, 0], 1e-12, "D=1 mean")


def test_layout_equivalence(coracle):
    rng = np.random.default_rng(8)
    x_cl = rng.normal(size=(2, 5, 3)).astype(np.float32)  # [N, D, C]
    dy_cl = rng.normal(size=(2, 5, 3)).astype(np.float32)
    gamma = rng.uniform(0.5, 1.5, size=3).astype(np.float32)
    beta = rng.normal(size=3).astype(np.float32)
    x_cf = np.ascontiguousarray(x_cl.transpose(0, 2, 1))
    dy_cf = np.ascontiguousarray(dy_cl.transpose(0, 2, 1))
    y1, m1, r1 = coracle.in_fwd(x_cl, gamma, beta, 1e-3, "f32", False)
    y2, m2, r2 = coracle.in_fwd(x_cf, gamma, beta, 1e-3, "f32", True)
    _close(y2.transpose(0, 2, 1), y1, 1e-12, "y")
    _close(m2, m1, 1e-12, "mean")
    _close(r2, r1, 1e-12, "inv_std")
    d1 = coracle.in_bwd(dy_cl, x_cl, gamma, m1, r1, "f32", False)
    d2 = coracle.in_bwd(dy_cf, x_cf, gamma, m2, r2, "f32", True)
    _close(d2[0].transpose(0, 2, 1), d1[0], 1e-12, "dx")
    _close(d2[1], d1[1], 1e-12, "dgamma")
    _close(d2[2], d1[2], 1e-12, "dbeta")
    # brute-force loops on the same tiny tensor
    for n in range(2):
        for c in range(3):
            v = x_cl[n, :, c].astype(np.float64)
            assert abs(m1[n, c] - v.mean()) < 1e-12
            assert abs(r1[n, c] - 1.0 / np.sqrt(v.var() + 1e-3)) < 1e-12


def test_half_and_bfloat_conversions(coracle):
    L = coracle.lib
    bits = np.arange(65536, dtype=np.uint16)
    ref16 = bits.view(np.float16).astype(np.float32)
    ref_bf = torch.from_numpy(bits.view(np.int16)).view(torch.bfloat16).to(torch.float32).numpy()
    for b in range(0, 65536, 7):  # every 7th pattern keeps the ctypes loop short
        h = L.oracle_half_to_float(int(b))
        e = float(ref16[b])
        assert (np.isnan(h) and np.isnan(e)) or h == e, (b, h, e)
        f = L.oracle_bf16_to_float(int(b))
        e = float(ref_bf[b])
        assert (np.isnan(f) and np.isnan(e)) or f == e, (b, f, e)
    rng = np.random.default_rng(9)
    vals = np.concatenate([
        rng.normal(size=3000).astype(np.float32),
        (rng.normal(size=2000) * 1e-6).astype(np.float32),      # subnormal halves
        (rng.normal(size=1000) * 3e4).astype(np.float32),       # near the fp16 overflow edge
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e-8, 5.96e-8, 2.98e-8, 6.1e-5], np.float32),
        ref16[np.isfinite(ref16)][::97] * np.float32(1.0 + 2 ** -12),  # ties and near-ties
    ])
    with np.errstate(over="ignore"):
        want16 = vals.astype(np.float16).view(np.uint16)
    want_bf = torch.from_numpy(vals).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    for v, w16, wbf in zip(vals, want16, want_bf):
        assert L.oracle_float_to_half(float(v)) == int(w16), (v, w16)
        assert L.oracle_float_to_bf16(float(v)) == int(wbf), (v, wbf)
    assert np.array_equal(O.f32_to_bf16_bits(vals), want_bf)
