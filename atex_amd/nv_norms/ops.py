"""Op-level Python surface, mirroring the reference's generated op wrappers
(atex/nv_norms/python/ops/nv_norm_ops.py:19-25, op definitions in
atex/nv_norms/cc/ops/norm_ops.cc:148-202):

    fused_layer_norm_op(x, scale, offset, axis=[-1], epsilon=0.001)
        -> (y, reserve_space_1 = mean, reserve_space_2 = inverse std)
    fused_layer_norm_grad_op(y_backprop, x, scale, reserve_space_1, reserve_space_2,
                             axis=[-1], epsilon=0.001)
        -> (x_backprop, scale_backprop, offset_backprop)
    fused_instance_norm_op(x, scale, offset, data_format="N...C", epsilon=0.001)
    fused_instance_norm_grad_op(y_backprop, x, scale, reserve_space_1, reserve_space_2,
                                data_format="N...C", epsilon=0.001)

TensorFlow is not part of this stack; tensors are torch tensors, used purely as owners of
memory and of the HIP stream.  Output allocation (the OpKernel's allocate_output /
allocate_temp) happens here; validation, axis packing and flattening happen in the C ABI
(atexn_fused_*), which raises InvalidArgumentError like the reference's OP_REQUIRES checks.
Tensors on a ROCm device run the HIP kernels; tensors in host memory run the library's CPU
kernels (the reference registers both, fused_layer_norm_op.cc:465-484), chosen by the device
of the tensors like a framework's kernel registry does.  Either way the arithmetic is the
library's: nothing here computes.
"""
from __future__ import annotations

import ctypes
from typing import Sequence

import torch

from . import _capi
from ._capi import InvalidArgumentError

_DTYPE_CODE = {
    torch.float32: _capi.ATEXN_F32,
    torch.float16: _capi.ATEXN_F16,
    torch.bfloat16: _capi.ATEXN_BF16,
}


def _code(t: torch.Tensor, name: str) -> int:
    try:
        return _DTYPE_CODE[t.dtype]
    except KeyError:
        raise InvalidArgumentError(_capi.ATEXN_INVALID_ARGUMENT,
                                   f"{name}: unsupported dtype {t.dtype}") from None


def _desc(t: torch.Tensor, name: str) -> _capi.AtexnTensor:
    if not t.is_contiguous():
        raise InvalidArgumentError(_capi.ATEXN_INVALID_ARGUMENT, f"{name} must be contiguous (row-major)")
    if t.is_cuda:
        device = _capi.ATEXN_DEVICE_GPU
    elif t.device.type == "cpu":
        device = _capi.ATEXN_DEVICE_CPU
    else:
        raise InvalidArgumentError(_capi.ATEXN_INVALID_ARGUMENT, f"{name}: unsupported device {t.device}")
    return _capi.make_tensor(_code(t, name), tuple(t.shape), t.data_ptr() if t.numel() else 0, device)


class _on_device:
    """Makes a GPU tensor's device current for the allocations and the call (the library plans
    for the current device); nothing to do for host tensors."""

    def __init__(self, t: torch.Tensor):
        self._ctx = torch.cuda.device(t.device) if t.is_cuda else None

    def __enter__(self):
        if self._ctx is not None:
            self._ctx.__enter__()

    def __exit__(self, *exc):
        if self._ctx is not None:
            return self._ctx.__exit__(*exc)
        return False


def _axis_array(axis) -> tuple:
    if isinstance(axis, int):
        axis = [axis]
    axis = [int(a) for a in axis]
    return (ctypes.c_int * max(len(axis), 1))(*axis), len(axis)


def _workspace(nbytes: int, device) -> tuple:
    if nbytes == 0:
        return None, None
    buf = torch.empty(nbytes, dtype=torch.uint8, device=device)
    return buf, buf.data_ptr()


def _stream(device) -> int:
    if device.type != "cuda":
        return 0
    return torch.cuda.current_stream(device).cuda_stream


def _prod(xs) -> int:
    p = 1
    for v in xs:
        p *= int(v)
    return p


def fused_layer_norm_op(x: torch.Tensor, scale: torch.Tensor, offset: torch.Tensor,
                        axis: Sequence[int] = (-1,), epsilon: float = 0.001):
    L = _capi.lib()
    ax, n_ax = _axis_array(axis)
    xd, sd, od = _desc(x, "x"), _desc(scale, "scale"), _desc(offset, "offset")
    n, d = ctypes.c_int64(), ctypes.c_int64()
    _capi.check(L.atexn_layer_norm_resolve_axes(xd.rank, xd.dims, ax, n_ax, ctypes.byref(n), ctypes.byref(d)))
    with _on_device(x):
        y = torch.empty_like(x)
        mean = torch.empty(n.value, dtype=torch.float32, device=x.device)
        inv_std = torch.empty(n.value, dtype=torch.float32, device=x.device)
        ws, ws_ptr = _workspace(L.atexn_fused_layer_norm_workspace_bytes(ctypes.byref(xd), ax, n_ax), x.device)
        yd, md, rd = _desc(y, "y"), _desc(mean, "mean"), _desc(inv_std, "inv_std")
        _capi.check(L.atexn_fused_layer_norm(
            ctypes.byref(xd), ctypes.byref(sd), ctypes.byref(od), float(epsilon), ax, n_ax,
            ctypes.byref(yd), ctypes.byref(md), ctypes.byref(rd), ws_ptr,
            0 if ws is None else ws.numel(), _stream(x.device)))
    return y, mean, inv_std


def fused_layer_norm_grad_op(y_backprop: torch.Tensor, x: torch.Tensor, scale: torch.Tensor,
                             reserve_space_1: torch.Tensor, reserve_space_2: torch.Tensor,
                             axis: Sequence[int] = (-1,), epsilon: float = 0.001):
    del epsilon  # attr of the op, unused by the gradient math (norm_ops.cc:172)
    L = _capi.lib()
    ax, n_ax = _axis_array(axis)
    dyd, xd, sd = _desc(y_backprop, "y_backprop"), _desc(x, "x"), _desc(scale, "scale")
    md, rd = _desc(reserve_space_1, "reserve_space_1"), _desc(reserve_space_2, "reserve_space_2")
    with _on_device(x):
        dx = torch.empty_like(x)
        # shaped like scale as passed in (fused_layer_norm_op.cc:451-457)
        dgamma = torch.empty(tuple(scale.shape), dtype=torch.float32, device=x.device)
        dbeta = torch.empty(tuple(scale.shape), dtype=torch.float32, device=x.device)
        ws, ws_ptr = _workspace(L.atexn_fused_layer_norm_grad_workspace_bytes(ctypes.byref(xd), ax, n_ax), x.device)
        dxd, dgd, dbd = _desc(dx, "x_backprop"), _desc(dgamma, "scale_backprop"), _desc(dbeta, "offset_backprop")
        _capi.check(L.atexn_fused_layer_norm_grad(
            ctypes.byref(dyd), ctypes.byref(xd), ctypes.byref(sd), ctypes.byref(md), ctypes.byref(rd),
            ax, n_ax, ctypes.byref(dxd), ctypes.byref(dgd), ctypes.byref(dbd), ws_ptr,
            0 if ws is None else ws.numel(), _stream(x.device)))
    return dx, dgamma, dbeta


def _fmt(data_format) -> bytes:
    if isinstance(data_format, bytes):
        return data_format
    return str(data_format).encode()


def fused_instance_norm_op(x: torch.Tensor, scale: torch.Tensor, offset: torch.Tensor,
                           data_format: str = "N...C", epsilon: float = 0.001):
    L = _capi.lib()
    fmt = _fmt(data_format)
    xd, sd, od = _desc(x, "x"), _desc(scale, "scale"), _desc(offset, "offset")
    layout = ctypes.c_int()
    n, c, d = ctypes.c_int64(), ctypes.c_int64(), ctypes.c_int64()
    _capi.check(L.atexn_instance_norm_resolve_format(xd.rank, xd.dims, fmt, ctypes.byref(layout),
                                                     ctypes.byref(n), ctypes.byref(c), ctypes.byref(d)))
    with _on_device(x):
        y = torch.empty_like(x)
        mean = torch.empty((n.value, c.value), dtype=torch.float32, device=x.device)
        inv_std = torch.empty((n.value, c.value), dtype=torch.float32, device=x.device)
        ws, ws_ptr = _workspace(L.atexn_fused_instance_norm_workspace_bytes(ctypes.byref(xd), fmt), x.device)
        yd, md, rd = _desc(y, "y"), _desc(mean, "mean"), _desc(inv_std, "inv_std")
        _capi.check(L.atexn_fused_instance_norm(
            ctypes.byref(xd), ctypes.byref(sd), ctypes.byref(od), float(epsilon), fmt,
            ctypes.byref(yd), ctypes.byref(md), ctypes.byref(rd), ws_ptr,
            0 if ws is None else ws.numel(), _stream(x.device)))
    return y, mean, inv_std


def fused_instance_norm_grad_op(y_backprop: torch.Tensor, x: torch.Tensor, scale: torch.Tensor,
                                reserve_space_1: torch.Tensor, reserve_space_2: torch.Tensor,
                                data_format: str = "N...C", epsilon: float = 0.001):
    del epsilon
    L = _capi.lib()
    fmt = _fmt(data_format)
    dyd, xd, sd = _desc(y_backprop, "y_backprop"), _desc(x, "x"), _desc(scale, "scale")
    md, rd = _desc(reserve_space_1, "reserve_space_1"), _desc(reserve_space_2, "reserve_space_2")
    with _on_device(x):
        dx = torch.empty_like(x)
        dgamma = torch.empty(tuple(scale.shape), dtype=torch.float32, device=x.device)
        dbeta = torch.empty(tuple(scale.shape), dtype=torch.float32, device=x.device)
        ws, ws_ptr = _workspace(L.atexn_fused_instance_norm_grad_workspace_bytes(ctypes.byref(xd), fmt), x.device)
        dxd, dgd, dbd = _desc(dx, "x_backprop"), _desc(dgamma, "scale_backprop"), _desc(dbeta, "offset_backprop")
        _capi.check(L.atexn_fused_instance_norm_grad(
            ctypes.byref(dyd), ctypes.byref(xd), ctypes.byref(sd), ctypes.byref(md), ctypes.byref(rd),
            fmt, ctypes.byref(dxd), ctypes.byref(dgd), ctypes.byref(dbd), ws_ptr,
            0 if ws is None else ws.numel(), _stream(x.device)))
    return dx, dgamma, dbeta
