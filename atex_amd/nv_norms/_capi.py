"""ctypes binding of libatex_norms_hip.so (the C ABI declared in include/atex_norms.h).

Fails loudly when the library is missing: nothing outside it computes (its CPU kernels serve
host tensors; they are no fallback for a GPU call).
"""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.normpath(os.path.join(_HERE, "..", "lib", "libatex_norms_hip.so"))

ATEXN_F32, ATEXN_F16, ATEXN_BF16 = 0, 1, 2
ATEXN_LAYOUT_NC_, ATEXN_LAYOUT_N_C = 0, 1
ATEXN_OK, ATEXN_INVALID_ARGUMENT, ATEXN_LAUNCH_ERROR = 0, 1, 2
ATEXN_DEVICE_GPU, ATEXN_DEVICE_CPU = 0, 1
ATEXN_MAX_RANK = 8


class AtexnTensor(ctypes.Structure):
    _fields_ = [
        ("dtype", ctypes.c_int),
        ("rank", ctypes.c_int),
        ("dims", ctypes.c_int64 * ATEXN_MAX_RANK),
        ("data", ctypes.c_void_p),
        ("device", ctypes.c_int),
    ]


class AtexnError(RuntimeError):
    """A non-OK status from the library. `.status` holds the code."""

    def __init__(self, status: int, message: str):
        super().__init__(message)
        self.status = status


class InvalidArgumentError(AtexnError, ValueError):
    """Mirror of TensorFlow's errors.InvalidArgumentError for this host."""


_lib = None

# name -> (restype, argtypes); every symbol that include/atex_norms.h declares
_vp, _i, _i64, _f, _sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_float, ctypes.c_size_t
_tp = ctypes.POINTER(AtexnTensor)
_ip = ctypes.POINTER(ctypes.c_int)
_i64p = ctypes.POINTER(ctypes.c_int64)
SIGNATURES = {
    "atexn_status_string": (ctypes.c_char_p, [_i]),
    "atexn_last_error": (ctypes.c_char_p, []),
    "atexn_abi_version": (_i, []),
    "atexn_layer_norm_fwd_workspace_bytes": (_sz, [_i, _i64, _i64]),
    "atexn_layer_norm_fwd": (_i, [_i, _vp, _vp, _vp, _i64, _i64, _f, _vp, _vp, _vp, _vp, _sz, _vp]),
    "atexn_layer_norm_bwd_workspace_bytes": (_sz, [_i, _i64, _i64]),
    "atexn_layer_norm_bwd": (_i, [_i, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _vp, _vp, _vp, _vp, _sz, _vp]),
    "atexn_layer_norm_bwd_static": (_i, [_i, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _vp, _vp, _vp, _vp]),
    "atexn_instance_norm_fwd_workspace_bytes": (_sz, [_i, _i, _i64, _i64, _i64]),
    "atexn_instance_norm_fwd": (_i, [_i, _i, _vp, _vp, _vp, _i64, _i64, _i64, _f, _vp, _vp, _vp, _vp, _sz, _vp]),
    "atexn_instance_norm_bwd_workspace_bytes": (_sz, [_i, _i, _i64, _i64, _i64]),
    "atexn_instance_norm_bwd": (_i, [_i, _i, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp, _vp, _vp, _vp, _sz, _vp]),
    "atexn_layer_norm_fwd_cpu": (_i, [_i, _vp, _vp, _vp, _i64, _i64, _f, _vp, _vp, _vp]),
    "atexn_layer_norm_bwd_cpu": (_i, [_i, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _vp, _vp, _vp]),
    "atexn_instance_norm_fwd_cpu": (_i, [_i, _i, _vp, _vp, _vp, _i64, _i64, _i64, _f, _vp, _vp, _vp]),
    "atexn_instance_norm_bwd_cpu": (_i, [_i, _i, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp, _vp, _vp]),
    "atexn_layer_norm_resolve_axes": (_i, [_i, _i64p, _ip, _i, _i64p, _i64p]),
    "atexn_instance_norm_resolve_format": (_i, [_i, _i64p, ctypes.c_char_p, _ip, _i64p, _i64p, _i64p]),
    "atexn_fused_layer_norm_workspace_bytes": (_sz, [_tp, _ip, _i]),
    "atexn_fused_layer_norm": (_i, [_tp, _tp, _tp, _f, _ip, _i, _tp, _tp, _tp, _vp, _sz, _vp]),
    "atexn_fused_layer_norm_grad_workspace_bytes": (_sz, [_tp, _ip, _i]),
    "atexn_fused_layer_norm_grad": (_i, [_tp, _tp, _tp, _tp, _tp, _ip, _i, _tp, _tp, _tp, _vp, _sz, _vp]),
    "atexn_fused_instance_norm_workspace_bytes": (_sz, [_tp, ctypes.c_char_p]),
    "atexn_fused_instance_norm": (_i, [_tp, _tp, _tp, _f, ctypes.c_char_p, _tp, _tp, _tp, _vp, _sz, _vp]),
    "atexn_fused_instance_norm_grad_workspace_bytes": (_sz, [_tp, ctypes.c_char_p]),
    "atexn_fused_instance_norm_grad": (_i, [_tp, _tp, _tp, _tp, _tp, ctypes.c_char_p, _tp, _tp, _tp, _vp, _sz, _vp]),
}
# the extra entry points of the benchmark build (csrc/bench_hooks.h)
BENCH_SIGNATURES = {
    "atexn_set_tuning": (_i, [ctypes.c_char_p, _i]),
    "atexn_bench_describe_bwd": (_i, [_i, _i, _i, _i64, _i64, _i64, ctypes.c_char_p, _sz]),
    "atexn_bench_mark_exchange_trouble": (_i, [_i]),
    "atexn_bench_exchange_trouble_age": (_i, []),
    "atexn_bench_occupy": (_i, [_i, ctypes.c_double, _vp]),
}
BENCH_LIB_PATH = LIB_PATH.replace(".so", "_bench.so")
_bench_lib = None


def lib() -> ctypes.CDLL:
    """Loads the library once; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python -m atex_amd.build` "
                "(there is no fallback implementation)")
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def bench_lib() -> ctypes.CDLL:
    """The benchmark build of the library: the same sources plus atexn_set_tuning (launch-planning
    parameters, process-wide) and atexn_bench_describe_bwd.  For bench.py and for tests that
    force a particular kernel family; the product path never loads it."""
    global _bench_lib
    if _bench_lib is None:
        if not os.path.exists(BENCH_LIB_PATH):
            raise ImportError(f"{BENCH_LIB_PATH} is missing: build it with `python -m atex_amd.build`")
        L = ctypes.CDLL(BENCH_LIB_PATH)
        for name, (res, args) in {**SIGNATURES, **BENCH_SIGNATURES}.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _bench_lib = L
    return _bench_lib


def check(status: int, L=None) -> None:
    if status == ATEXN_OK:
        return
    L = L or lib()
    msg = L.atexn_last_error().decode("utf-8", "replace")
    name = L.atexn_status_string(status).decode()
    if status == ATEXN_INVALID_ARGUMENT:
        raise InvalidArgumentError(status, f"{name}: {msg}")
    raise AtexnError(status, f"{name}: {msg}")


_Dims = ctypes.c_int64 * ATEXN_MAX_RANK


def make_tensor(dtype_code: int, shape, ptr: int, device: int = ATEXN_DEVICE_GPU) -> AtexnTensor:
    if len(shape) > ATEXN_MAX_RANK:
        raise InvalidArgumentError(ATEXN_INVALID_ARGUMENT, f"rank {len(shape)} > {ATEXN_MAX_RANK}")
    # one constructor call: field-by-field assignment costs several microseconds per tensor
    return AtexnTensor(dtype_code, len(shape), _Dims(*shape), ptr if ptr else None, device)
