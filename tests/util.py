"""Shared helpers of the test-suite: seeded inputs of the benchmark configurations,
storage-dtype conversions, tolerances and the kernel-level C-ABI call wrappers."""
from __future__ import annotations

import ctypes

import numpy as np

from oracle import oracle as O

# Tolerances.  The acceptance bar is fp32 rtol 1e-5; fp16 / bf16 rtol 1e-2 on y and dx, 1e-3 on
# the fp32 dgamma / dbeta.  The tests hold the kernels to much less, which is what arithmetic in
# float32 on the already-rounded inputs delivers:
#   * y, dx in fp16 / bf16: within one unit in the last place of the STORAGE type of the float64
#     reference (half an ulp from the final rounding, the rest for float32 results that straddle
#     a rounding boundary), plus a float32-sized absolute term for results near zero;
#   * saved statistics: float32 accuracy whatever the storage type (1e-5, as for fp32 inputs);
#   * dgamma / dbeta: 1e-4 (float32 sums of up to a few hundred thousand terms).
# Plain float entries mean |got - ref| <= rtol * |ref| + rtol * rms(ref): the absolute term covers
# results near zero.
class Ulp:
    """|got - ref| <= ulps * ulp_storage(ref) + floor * max(rms(ref), scale)."""

    def __init__(self, storage, ulps=1.01, floor=4e-6):
        self.storage, self.ulps, self.floor = storage, ulps, floor

    def bound(self, ref, rms):
        mant, emin = (10, -14) if self.storage == "f16" else (7, -126)
        with np.errstate(divide="ignore"):
            e = np.floor(np.log2(np.maximum(np.abs(ref), 2.0 ** emin)))
        return self.ulps * np.exp2(e - mant) + self.floor * rms


TOL = {
    "f32": dict(y=1e-5, stat=1e-5, dx=1e-5, dw=1e-5),
    "f16": dict(y=Ulp("f16"), stat=1e-5, dx=Ulp("f16"), dw=1e-4),
    "bf16": dict(y=Ulp("bf16"), stat=1e-5, dx=Ulp("bf16"), dw=1e-4),
}


def assert_close(got, ref, rtol, what="", scale=0.0):
    """`rtol`: a float (relative + rms-scaled absolute bound) or an Ulp bound.
    `scale`: magnitude of the terms the result is a difference of, when that is larger
    than the result itself (dx is r*g minus its projections; for a one-element row the
    exact answer is 0 and only rounding residue is left)."""
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape, (what, got.shape, ref.shape)
    if ref.size == 0:
        return
    assert np.all(np.isfinite(got)), f"{what}: non-finite values"
    rms = max(float(np.sqrt(np.mean(ref * ref))), float(scale))
    if isinstance(rtol, Ulp):
        bound = rtol.bound(ref, rms)
    else:
        bound = rtol * np.abs(ref) + rtol * rms
    err = np.abs(got - ref)
    worst = int(np.argmax(err - bound))
    assert np.all(err <= bound), (
        f"{what}: max err {err.max():.3e} (rms(ref) {rms:.3e}); worst at flat index {worst}: "
        f"got {got.flat[worst]!r} ref {ref.flat[worst]!r} bound {bound.flat[worst]:.3e}")


def dx_scale(dy, gamma_rms, rstd, dtype):
    """rms of r * dy * gamma, the leading term of dx."""
    d = O.from_storage(dy, dtype)
    return float(np.sqrt(np.mean(d * d))) * float(gamma_rms) * float(np.sqrt(np.mean(np.square(rstd))))


# ------------------------------------------------------------------ seeded inputs
def rng_for(cfg_index: int):
    return np.random.Generator(np.random.PCG64(1000 + cfg_index))


def affine_params(rng, d):
    gamma = rng.uniform(0.5, 1.5, size=d).astype(np.float32)
    beta = (rng.standard_normal(d) * 0.1).astype(np.float32)
    return gamma, beta


def ln_inputs(cfg: str, N: int, D: int, dtype: str, seed_index: int):
    """cfg in {'plain', 'row_mean', 'scaled_rows'} (configs[0], [1], [2])."""
    rng = rng_for(seed_index)
    x = rng.standard_normal((N, D), dtype=np.float32)
    if cfg == "row_mean":
        x += rng.uniform(-2, 2, size=(N, 1)).astype(np.float32)
    elif cfg == "scaled_rows":
        x[rng.random(N) < 0.01] *= 10.0
    gamma, beta = affine_params(rng, D)
    dy = rng.standard_normal((N, D), dtype=np.float32)
    return O.to_storage(x, dtype), gamma, beta, O.to_storage(dy, dtype)


def in_inputs(N: int, C: int, spatial: int, dtype: str, channel_first: bool, seed_index: int,
              stddev: float = 1.0):
    """x ~ N(0, stddev) + per-channel offset U(-1,1), generated channels-last; the
    channel-first variant is the transpose of the same values."""
    rng = rng_for(seed_index)
    x = rng.standard_normal((N, spatial, C), dtype=np.float32) * np.float32(stddev)
    x += rng.uniform(-1, 1, size=(1, 1, C)).astype(np.float32)
    gamma, beta = affine_params(rng, C)
    dy = rng.standard_normal((N, spatial, C), dtype=np.float32)
    if channel_first:
        x = np.ascontiguousarray(np.transpose(x, (0, 2, 1)))
        dy = np.ascontiguousarray(np.transpose(dy, (0, 2, 1)))
    return O.to_storage(x, dtype), gamma, beta, O.to_storage(dy, dtype)


# ---------------------------------------------------------------- torch <-> numpy
def torch_dtype(dtype: str):
    import torch

    return {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[dtype]


def to_device(a: np.ndarray, dtype: str, device="cuda:0"):
    """numpy storage array (bf16 as uint16 bits) -> torch tensor on the device."""
    import torch

    if dtype == "bf16":
        return torch.from_numpy(a.view(np.int16)).to(device).view(torch.bfloat16)
    return torch.from_numpy(a).to(device)


def misalign(t, elements: int = 1):
    """A copy of t whose storage starts `elements` elements past an allocation boundary, so
    that no row, vector or parameter array is 16-byte aligned."""
    import torch

    buf = torch.empty(t.numel() + elements, dtype=t.dtype, device=t.device)
    v = buf[elements:].view(t.shape)
    v.copy_(t)
    assert v.data_ptr() % 16 != 0 or t.numel() == 0
    return v


def to_host(t, dtype: str | None = None) -> np.ndarray:
    """torch tensor -> float64 numpy values."""
    import torch

    t = t.detach()
    if t.dtype == torch.bfloat16:
        return O.bf16_bits_to_f32(t.view(torch.int16).cpu().numpy().view(np.uint16)).astype(np.float64)
    return t.cpu().numpy().astype(np.float64)


# ------------------------------------------------------------ kernel-level C ABI
class Capi:
    """Calls the kernel-level entry points of libatex_norms_hip.so on torch device memory.
    bench=True: through the benchmark build of the library instead, the only one whose launch
    planning can be changed (atexn_set_tuning), for tests that force a kernel family."""

    def __init__(self, bench=False):
        import torch

        from atex_amd.nv_norms import _capi

        self.torch = torch
        self.capi = _capi
        self.L = _capi.bench_lib() if bench else _capi.lib()

    def _check(self, status):
        self.capi.check(status, self.L)

    def _ws(self, nbytes, device):
        if nbytes == 0:
            return None, None, 0
        buf = self.torch.empty(nbytes, dtype=self.torch.uint8, device=device)
        return buf, buf.data_ptr(), nbytes

    @staticmethod
    def _p(t):
        return t.data_ptr() if t is not None and t.numel() else None

    def _stream(self, device):
        return self.torch.cuda.current_stream(device).cuda_stream

    def ln_fwd(self, x, gamma, beta, eps, dtype, y=None):
        t = self.torch
        N, D = x.shape
        code = O.DTYPE_CODE[dtype]
        y = t.empty_like(x) if y is None else y
        mean = t.empty(N, dtype=t.float32, device=x.device)
        rstd = t.empty(N, dtype=t.float32, device=x.device)
        ws, wp, wb = self._ws(self.L.atexn_layer_norm_fwd_workspace_bytes(code, N, D), x.device)
        self._check(self.L.atexn_layer_norm_fwd(
            code, self._p(x), self._p(gamma), self._p(beta), N, D, eps, self._p(y), self._p(mean),
            self._p(rstd), wp, wb, self._stream(x.device)))
        return y, mean, rstd

    def ln_bwd(self, dy, x, gamma, mean, rstd, dtype, dx=None):
        t = self.torch
        N, D = x.shape
        code = O.DTYPE_CODE[dtype]
        dx = t.empty_like(x) if dx is None else dx
        dg = t.empty(D, dtype=t.float32, device=x.device)
        db = t.empty(D, dtype=t.float32, device=x.device)
        ws, wp, wb = self._ws(self.L.atexn_layer_norm_bwd_workspace_bytes(code, N, D), x.device)
        self._check(self.L.atexn_layer_norm_bwd(
            code, self._p(dy), self._p(x), self._p(gamma), self._p(mean), self._p(rstd), N, D,
            self._p(dx), self._p(dg), self._p(db), wp, wb, self._stream(x.device)))
        return dx, dg, db

    @staticmethod
    def _ncd(shape, channel_first):
        return (shape[0], shape[1], shape[2]) if channel_first else (shape[0], shape[2], shape[1])

    def in_fwd(self, x, gamma, beta, eps, dtype, channel_first, y=None):
        t = self.torch
        N, C, D = self._ncd(x.shape, channel_first)
        code = O.DTYPE_CODE[dtype]
        layout = 0 if channel_first else 1
        y = t.empty_like(x) if y is None else y
        mean = t.empty((N, C), dtype=t.float32, device=x.device)
        rstd = t.empty((N, C), dtype=t.float32, device=x.device)
        ws, wp, wb = self._ws(self.L.atexn_instance_norm_fwd_workspace_bytes(code, layout, N, C, D), x.device)
        self._check(self.L.atexn_instance_norm_fwd(
            code, layout, self._p(x), self._p(gamma), self._p(beta), N, C, D, eps, self._p(y),
            self._p(mean), self._p(rstd), wp, wb, self._stream(x.device)))
        return y, mean, rstd

    def in_bwd(self, dy, x, gamma, mean, rstd, dtype, channel_first, dx=None):
        t = self.torch
        N, C, D = self._ncd(x.shape, channel_first)
        code = O.DTYPE_CODE[dtype]
        layout = 0 if channel_first else 1
        dx = t.empty_like(x) if dx is None else dx
        dg = t.empty(C, dtype=t.float32, device=x.device)
        db = t.empty(C, dtype=t.float32, device=x.device)
        ws, wp, wb = self._ws(self.L.atexn_instance_norm_bwd_workspace_bytes(code, layout, N, C, D), x.device)
        self._check(self.L.atexn_instance_norm_bwd(
            code, layout, self._p(dy), self._p(x), self._p(gamma), self._p(mean), self._p(rstd),
            N, C, D, self._p(dx), self._p(dg), self._p(db), wp, wb, self._stream(x.device)))
        return dx, dg, db
