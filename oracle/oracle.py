"""Python face of the CPU oracle (TEST INFRASTRUCTURE ONLY).

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this
module.  It offers two independent restatements of the reference's algorithm:

* ``*_np``  -- vectorised numpy float64 closed forms, following the reference CPU
  functors (atex/nv_norms/cc/kernels/fused_layer_norm_op.cc:27-223,
  fused_instance_norm_op.cc:39-284);
* ``COracle`` -- ctypes binding of ``libnorms_oracle.so`` (norms_oracle.c), the
  plain-C restatement in float (reference arithmetic, also the timed CPU baseline)
  and double (ground truth for the parity tests).

Storage dtypes are named "f32", "f16", "bf16".  bfloat16 arrays are carried as
numpy uint16 bit patterns (numpy has no bfloat16).
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libnorms_oracle.so")

DTYPE_CODE = {"f32": 0, "f16": 1, "bf16": 2}


# --------------------------------------------------------------------------- bf16
def f32_to_bf16_bits(a: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even float32 -> bfloat16 bit patterns (uint16)."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
    lsb = (u >> 16) & 1
    return ((u + 0x7FFF + lsb) >> 16).astype(np.uint16)


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def to_storage(a: np.ndarray, dtype: str) -> np.ndarray:
    """Round a float array to the storage dtype's in-memory representation."""
    if dtype == "f32":
        return np.ascontiguousarray(a, dtype=np.float32)
    if dtype == "f16":
        return np.ascontiguousarray(a).astype(np.float16)
    if dtype == "bf16":
        return f32_to_bf16_bits(np.asarray(a, dtype=np.float32))
    raise ValueError(dtype)


def from_storage(a: np.ndarray, dtype: str) -> np.ndarray:
    """Storage representation -> float64 values."""
    if dtype == "bf16":
        return bf16_bits_to_f32(a).astype(np.float64)
    return np.asarray(a).astype(np.float64)


# --------------------------------------------------------------- numpy closed forms
def ln_fwd_np(x, gamma, beta, eps):
    """x [N, D] float64 -> (y, mean[N], inv_std[N]); biased variance (LN.cc:66-81)."""
    x = np.asarray(x, dtype=np.float64)
    mean = x.mean(axis=1)
    xc = x - mean[:, None]
    var = (xc * xc).mean(axis=1)
    inv_std = 1.0 / np.sqrt(var + eps)
    y = xc * inv_std[:, None] * np.asarray(gamma, np.float64)[None, :] + np.asarray(beta, np.float64)[None, :]
    return y, mean, inv_std


def ln_bwd_np(dy, x, gamma, mean, inv_std):
    """(dx, dgamma, dbeta) from the saved statistics (LN.cc:160-221)."""
    dy = np.asarray(dy, np.float64)
    x = np.asarray(x, np.float64)
    g = np.asarray(gamma, np.float64)[None, :]
    m = np.asarray(mean, np.float64)[:, None]
    r = np.asarray(inv_std, np.float64)[:, None]
    D = x.shape[1]
    xc = x - m
    dgamma = (dy * xc * r).sum(axis=0)
    dbeta = dy.sum(axis=0)
    dl_dx = dy * g * r
    dl_dvar = (dl_dx * xc * (-0.5) * r * r).sum(axis=1, keepdims=True)
    dl_dmean = (-dl_dx).sum(axis=1, keepdims=True) + (dl_dvar * (-2.0 / D) * xc).sum(axis=1, keepdims=True)
    dx = dl_dx + dl_dvar * (2.0 * xc / D) + dl_dmean / D
    return dx, dgamma, dbeta


def _in_view(a, channel_first):
    """[N,C,D] or [N,D,C] -> [N,C,D] float64 view."""
    a = np.asarray(a, np.float64)
    return a if channel_first else np.transpose(a, (0, 2, 1))


def in_fwd_np(x, gamma, beta, eps, channel_first):
    """x [N,C,D] (channel_first) or [N,D,C] -> (y same layout, mean[N,C], inv_std[N,C])."""
    xv = _in_view(x, channel_first)
    mean = xv.mean(axis=2)
    xc = xv - mean[:, :, None]
    var = (xc * xc).mean(axis=2)
    inv_std = 1.0 / np.sqrt(var + eps)
    g = np.asarray(gamma, np.float64)[None, :, None]
    b = np.asarray(beta, np.float64)[None, :, None]
    y = xc * inv_std[:, :, None] * g + b
    if not channel_first:
        y = np.transpose(y, (0, 2, 1))
    return np.ascontiguousarray(y), mean, inv_std


def in_bwd_np(dy, x, gamma, mean, inv_std, channel_first):
    dyv = _in_view(dy, channel_first)
    xv = _in_view(x, channel_first)
    D = xv.shape[2]
    g = np.asarray(gamma, np.float64)[None, :, None]
    m = np.asarray(mean, np.float64)[:, :, None]
    r = np.asarray(inv_std, np.float64)[:, :, None]
    xc = xv - m
    dgamma = (dyv * xc * r).sum(axis=(0, 2))
    dbeta = dyv.sum(axis=(0, 2))
    dl_dx = dyv * g * r
    dl_dvar = (dl_dx * xc * (-0.5) * r * r).sum(axis=2, keepdims=True)
    dl_dmean = (-dl_dx).sum(axis=2, keepdims=True) + (dl_dvar * (-2.0 / D) * xc).sum(axis=2, keepdims=True)
    dx = dl_dx + dl_dvar * (2.0 * xc / D) + dl_dmean / D
    if not channel_first:
        dx = np.transpose(dx, (0, 2, 1))
    return np.ascontiguousarray(dx), dgamma, dbeta


# ------------------------------------------------------------------------ C oracle
def build(force: bool = False) -> str:
    """Compile libnorms_oracle.so with gcc (idempotent unless force)."""
    src = os.path.join(_HERE, "norms_oracle.c")
    if force or not os.path.exists(LIB_PATH) or os.path.getmtime(LIB_PATH) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libnorms_oracle.so"], stdout=subprocess.DEVNULL)
    return LIB_PATH


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


class COracle:
    """ctypes binding of norms_oracle.c.  Inputs are numpy arrays in storage dtype."""

    def __init__(self, path: str | None = None):
        path = path or LIB_PATH
        if not os.path.exists(path):
            build()
        self.lib = ctypes.CDLL(path)
        L = self.lib
        vp, i64, f, d, i = ctypes.c_void_p, ctypes.c_int64, ctypes.c_float, ctypes.c_double, ctypes.c_int
        L.oracle_ln_fwd_f32.argtypes = [i, vp, vp, vp, i64, i64, f, vp, vp, vp]
        L.oracle_ln_fwd_f64.argtypes = [i, vp, vp, vp, i64, i64, d, vp, vp, vp]
        L.oracle_ln_bwd_f32.argtypes = [i, vp, vp, vp, vp, vp, i64, i64, vp, vp, vp]
        L.oracle_ln_bwd_f64.argtypes = [i, vp, vp, vp, vp, vp, i64, i64, vp, vp, vp]
        L.oracle_in_fwd_f32.argtypes = [i, i, vp, vp, vp, i64, i64, i64, f, vp, vp, vp]
        L.oracle_in_fwd_f64.argtypes = [i, i, vp, vp, vp, i64, i64, i64, d, vp, vp, vp]
        L.oracle_in_bwd_f32.argtypes = [i, i, vp, vp, vp, vp, vp, i64, i64, i64, vp, vp, vp]
        L.oracle_in_bwd_f64.argtypes = [i, i, vp, vp, vp, vp, vp, i64, i64, i64, vp, vp, vp]
        for n in ("oracle_ln_fwd_f32", "oracle_ln_fwd_f64", "oracle_ln_bwd_f32", "oracle_ln_bwd_f64",
                  "oracle_in_fwd_f32", "oracle_in_fwd_f64", "oracle_in_bwd_f32", "oracle_in_bwd_f64"):
            getattr(L, n).restype = None
        L.oracle_half_to_float.argtypes = [ctypes.c_uint16]
        L.oracle_half_to_float.restype = f
        L.oracle_float_to_half.argtypes = [f]
        L.oracle_float_to_half.restype = ctypes.c_uint16
        L.oracle_bf16_to_float.argtypes = [ctypes.c_uint16]
        L.oracle_bf16_to_float.restype = f
        L.oracle_float_to_bf16.argtypes = [f]
        L.oracle_float_to_bf16.restype = ctypes.c_uint16
        L.oracle_num_threads.restype = i
        L.oracle_set_num_threads.argtypes = [i]

    # -- helpers
    @staticmethod
    def _st(a, dtype):
        want = {"f32": np.float32, "f16": np.float16, "bf16": np.uint16}[dtype]
        a = np.ascontiguousarray(a)
        assert a.dtype == want, (a.dtype, dtype)
        return a

    @staticmethod
    def _f32(a):
        return np.ascontiguousarray(a, dtype=np.float32)

    def num_threads(self):
        return int(self.lib.oracle_num_threads())

    def set_num_threads(self, n):
        self.lib.oracle_set_num_threads(int(n))

    # -- LayerNorm
    def ln_fwd(self, x, gamma, beta, eps, dtype, f64=True):
        x = self._st(x, dtype)
        N, D = x.shape
        gamma, beta = self._f32(gamma), self._f32(beta)
        if f64:
            y = np.empty((N, D), np.float64); mean = np.empty(N, np.float64); rstd = np.empty(N, np.float64)
            self.lib.oracle_ln_fwd_f64(DTYPE_CODE[dtype], _p(x), _p(gamma), _p(beta), N, D, float(eps), _p(y), _p(mean), _p(rstd))
        else:
            y = np.empty_like(x); mean = np.empty(N, np.float32); rstd = np.empty(N, np.float32)
            self.lib.oracle_ln_fwd_f32(DTYPE_CODE[dtype], _p(x), _p(gamma), _p(beta), N, D, float(eps), _p(y), _p(mean), _p(rstd))
        return y, mean, rstd

    def ln_bwd(self, dy, x, gamma, mean, inv_std, dtype, f64=True):
        x = self._st(x, dtype); dy = self._st(dy, dtype)
        N, D = x.shape
        gamma = self._f32(gamma)
        if f64:
            mean = np.ascontiguousarray(mean, np.float64); inv_std = np.ascontiguousarray(inv_std, np.float64)
            dx = np.empty((N, D), np.float64); dg = np.empty(D, np.float64); db = np.empty(D, np.float64)
            self.lib.oracle_ln_bwd_f64(DTYPE_CODE[dtype], _p(dy), _p(x), _p(gamma), _p(mean), _p(inv_std), N, D, _p(dx), _p(dg), _p(db))
        else:
            mean = self._f32(mean); inv_std = self._f32(inv_std)
            dx = np.empty_like(x); dg = np.empty(D, np.float32); db = np.empty(D, np.float32)
            self.lib.oracle_ln_bwd_f32(DTYPE_CODE[dtype], _p(dy), _p(x), _p(gamma), _p(mean), _p(inv_std), N, D, _p(dx), _p(dg), _p(db))
        return dx, dg, db

    # -- InstanceNorm; x is [N,C,D] if channel_first else [N,D,C]
    @staticmethod
    def _ncd(shape, channel_first):
        return (shape[0], shape[1], shape[2]) if channel_first else (shape[0], shape[2], shape[1])

    def in_fwd(self, x, gamma, beta, eps, dtype, channel_first, f64=True):
        x = self._st(x, dtype)
        N, C, D = self._ncd(x.shape, channel_first)
        gamma, beta = self._f32(gamma), self._f32(beta)
        cf = 1 if channel_first else 0
        if f64:
            y = np.empty(x.shape, np.float64); mean = np.empty((N, C), np.float64); rstd = np.empty((N, C), np.float64)
            self.lib.oracle_in_fwd_f64(DTYPE_CODE[dtype], cf, _p(x), _p(gamma), _p(beta), N, C, D, float(eps), _p(y), _p(mean), _p(rstd))
        else:
            y = np.empty_like(x); mean = np.empty((N, C), np.float32); rstd = np.empty((N, C), np.float32)
            self.lib.oracle_in_fwd_f32(DTYPE_CODE[dtype], cf, _p(x), _p(gamma), _p(beta), N, C, D, float(eps), _p(y), _p(mean), _p(rstd))
        return y, mean, rstd

    def in_bwd(self, dy, x, gamma, mean, inv_std, dtype, channel_first, f64=True):
        x = self._st(x, dtype); dy = self._st(dy, dtype)
        N, C, D = self._ncd(x.shape, channel_first)
        gamma = self._f32(gamma)
        cf = 1 if channel_first else 0
        if f64:
            mean = np.ascontiguousarray(mean, np.float64); inv_std = np.ascontiguousarray(inv_std, np.float64)
            dx = np.empty(x.shape, np.float64); dg = np.empty(C, np.float64); db = np.empty(C, np.float64)
            self.lib.oracle_in_bwd_f64(DTYPE_CODE[dtype], cf, _p(dy), _p(x), _p(gamma), _p(mean), _p(inv_std), N, C, D, _p(dx), _p(dg), _p(db))
        else:
            mean = self._f32(mean); inv_std = self._f32(inv_std)
            dx = np.empty_like(x); dg = np.empty(C, np.float32); db = np.empty(C, np.float32)
            self.lib.oracle_in_bwd_f32(DTYPE_CODE[dtype], cf, _p(dy), _p(x), _p(gamma), _p(mean), _p(inv_std), N, C, D, _p(dx), _p(dg), _p(db))
        return dx, dg, db
