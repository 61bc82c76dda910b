"""The op-level surface and the layers on the GPU, written after the reference's own tests:
tests/fused_layer_norm_test.py (axis cases :250-260, dtype/shape sweeps :146-247, gradient
shape check :137-140, empty input :153-164) and tests/fused_instance_norm_test.py
(:93-123 op vs numpy, :125-143 layer, :145-199 sweeps).  Expected values come from the
numpy closed forms in float64 and, for the layers, from torch's own float32 kernels on the
same device."""
import numpy as np
import pytest

from oracle import oracle as O
from tests import util
from tests.util import TOL, assert_close

pytestmark = pytest.mark.gpu

EPS = 1e-3


def _np(t):
    return util.to_host(t)


def _rand(shape, dtype, seed):
    import torch

    rng = util.rng_for(seed)
    x = rng.standard_normal(shape, dtype=np.float32)
    return util.to_device(O.to_storage(x, dtype), dtype), rng


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("axis", [[1, 2], [-2, -1], [1, -1], [-2, 2], [-1], -1, [0, 1, 2]])
def test_layer_norm_op_axes(axis, dtype):
    import torch

    from atex_amd import nv_norms

    shape = (6, 10, 24)
    print(f"op LN axis={axis} dtype={dtype} shape={shape}", flush=True)
    x, rng = _rand(shape, dtype, 40)
    dy, _ = _rand(shape, dtype, 41)
    ax = [axis] if isinstance(axis, int) else axis
    ax = sorted(set(a % 3 for a in ax))
    wshape = tuple(shape[a] for a in ax)
    D = int(np.prod(wshape))
    N = int(np.prod(shape)) // D
    gamma = rng.uniform(0.5, 1.5, size=wshape).astype(np.float32)
    beta = (rng.standard_normal(wshape) * 0.1).astype(np.float32)
    gd, bd = torch.from_numpy(gamma).cuda(), torch.from_numpy(beta).cuda()

    y, mean, rstd = nv_norms.fused_layer_norm_op(x, gd, bd, axis=axis, epsilon=EPS)
    assert y.shape == x.shape and y.dtype == x.dtype
    assert mean.shape == (N,) and rstd.shape == (N,) and mean.dtype == torch.float32
    dx, dg, db = nv_norms.fused_layer_norm_grad_op(dy, x, gd, mean, rstd, axis=axis, epsilon=EPS)
    # the gradient of scale / offset has the SHAPE of scale (fused_layer_norm_test.py:137-140)
    assert dx.shape == x.shape and dg.shape == gd.shape and db.shape == bd.shape
    torch.cuda.synchronize()

    x64 = _np(x).reshape(N, D)
    y_ref, m_ref, r_ref = O.ln_fwd_np(x64, gamma.reshape(-1), beta.reshape(-1), EPS)
    dx_ref, dg_ref, db_ref = O.ln_bwd_np(_np(dy).reshape(N, D), x64, gamma.reshape(-1), _np(mean), _np(rstd))
    tol = TOL[dtype]
    assert_close(_np(y).reshape(N, D), y_ref, tol["y"], "y")
    assert_close(_np(mean), m_ref, tol["stat"], "mean")
    assert_close(_np(rstd), r_ref, tol["stat"], "inv_std")
    assert_close(_np(dx).reshape(N, D), dx_ref, tol["dx"], "dx")
    assert_close(_np(dg).reshape(-1), dg_ref, tol["dw"], "dgamma")
    assert_close(_np(db).reshape(-1), db_ref, tol["dw"], "dbeta")


def test_layer_norm_op_errors():
    import torch

    from atex_amd import nv_norms
    from atex_amd.nv_norms import InvalidArgumentError

    x = torch.zeros(4, 6, 8, device="cuda")
    g = torch.ones(48, device="cuda")
    with pytest.raises(InvalidArgumentError, match="axis is not packed from last dim."):
        nv_norms.fused_layer_norm_op(x, g, g, axis=[1])
    with pytest.raises(InvalidArgumentError, match="axis contains invalid value: 3"):
        nv_norms.fused_layer_norm_op(x, g, g, axis=[3])
    with pytest.raises(InvalidArgumentError, match="got 47 and 48"):
        nv_norms.fused_layer_norm_op(x, g, torch.ones(47, device="cuda"), axis=[1, 2])
    with pytest.raises(InvalidArgumentError, match="must be float32"):
        nv_norms.fused_layer_norm_op(x, g.half(), g, axis=[1, 2])
    with pytest.raises(InvalidArgumentError, match="unsupported dtype"):
        nv_norms.fused_layer_norm_op(x.double(), g, g, axis=[1, 2])
    with pytest.raises(InvalidArgumentError, match="contiguous"):
        nv_norms.fused_layer_norm_op(x.transpose(0, 1), g, g, axis=[1, 2])
    with pytest.raises(InvalidArgumentError, match="same device"):
        nv_norms.fused_layer_norm_op(x.cpu(), g, g, axis=[1, 2])
    y, m, r = nv_norms.fused_layer_norm_op(x, g, g, axis=[1, 2])
    with pytest.raises(InvalidArgumentError, match="x and y_backprop must have same shape"):
        nv_norms.fused_layer_norm_grad_op(torch.zeros(4, 6, 7, device="cuda"), x, g, m, r, axis=[1, 2])
    with pytest.raises(InvalidArgumentError, match="got 3 and 4"):
        nv_norms.fused_layer_norm_grad_op(x, x, g, m, r[:3].contiguous(), axis=[1, 2])


def test_instance_norm_op_errors():
    import torch

    from atex_amd import nv_norms
    from atex_amd.nv_norms import InvalidArgumentError

    x = torch.zeros(2, 8, 8, 32, device="cuda")
    g = torch.ones(32, device="cuda")
    with pytest.raises(InvalidArgumentError, match="We only accept 'NC...' or 'N...C' data format"):
        nv_norms.fused_instance_norm_op(x, g, g, data_format="NHW")
    with pytest.raises(InvalidArgumentError, match="input must be at least 4-dimensional"):
        nv_norms.fused_instance_norm_op(x[0], g, g)
    with pytest.raises(InvalidArgumentError, match="got 32 and 8"):
        nv_norms.fused_instance_norm_op(x, g, g, data_format="NC...")
    with pytest.raises(InvalidArgumentError, match="scale must be 1-dimensional"):
        nv_norms.fused_instance_norm_op(x, g.reshape(4, 8), g)
    with pytest.raises(InvalidArgumentError, match="same device"):
        nv_norms.fused_instance_norm_op(x.cpu(), g, g)


def test_empty_inputs():
    """fused_layer_norm_test.py:153-164: x of shape [0, 0]: empty y, no error; the weight
    gradients of an empty batch are zeros."""
    import torch

    from atex_amd import nv_norms

    x = torch.zeros(0, 0, device="cuda")
    g = torch.zeros(0, device="cuda")
    y, m, r = nv_norms.fused_layer_norm_op(x, g, g, axis=[-1])
    assert y.shape == (0, 0) and m.shape == (0,) and r.shape == (0,)
    x = torch.zeros(0, 16, device="cuda", dtype=torch.float16)
    g = torch.ones(16, device="cuda")
    y, m, r = nv_norms.fused_layer_norm_op(x, g, g)
    dx, dg, db = nv_norms.fused_layer_norm_grad_op(x, x, g, m, r)
    torch.cuda.synchronize()
    assert dx.shape == (0, 16) and float(dg.abs().sum()) == 0.0 and float(db.abs().sum()) == 0.0
    for fmt, shape in (("N...C", (0, 4, 4, 8)), ("NC...", (0, 8, 4, 4)), ("NDHWC", (2, 0, 4, 4, 8))):
        x = torch.zeros(shape, device="cuda")
        g = torch.ones(8, device="cuda")
        y, m, r = nv_norms.fused_instance_norm_op(x, g, g, data_format=fmt)
        assert y.shape == x.shape and m.shape == (shape[0], 8)
        dx, dg, db = nv_norms.fused_instance_norm_grad_op(x, x, g, m, r, data_format=fmt)
        torch.cuda.synchronize()
        assert dx.shape == x.shape and float(dg.abs().sum()) == 0.0 and float(db.abs().sum()) == 0.0


@pytest.mark.parametrize("dtype", ["f32", "f16"])
@pytest.mark.parametrize("fmt,shape", [
    ("N...C", (2, 6, 7, 24)), ("NC...", (2, 24, 6, 7)), ("NHWC", (2, 8, 8, 32)), ("NCHW", (2, 32, 8, 8)),
    ("NDHWC", (2, 4, 5, 6, 16)), ("NCDHW", (2, 16, 4, 5, 6)), ("N...C", (1, 3, 3, 3, 3, 8)),
])
def test_instance_norm_op(fmt, shape, dtype):
    import torch

    from atex_amd import nv_norms

    print(f"op IN fmt={fmt} shape={shape} dtype={dtype}", flush=True)
    cf = fmt[1] == "C"
    N, C = shape[0], (shape[1] if cf else shape[-1])
    D = int(np.prod(shape)) // (N * C)
    x, rng = _rand(shape, dtype, 50)
    dy, _ = _rand(shape, dtype, 51)
    gamma, beta = util.affine_params(rng, C)
    gd, bd = torch.from_numpy(gamma).cuda(), torch.from_numpy(beta).cuda()
    y, mean, rstd = nv_norms.fused_instance_norm_op(x, gd, bd, data_format=fmt, epsilon=EPS)
    assert y.shape == x.shape and mean.shape == (N, C) and rstd.shape == (N, C)
    dx, dg, db = nv_norms.fused_instance_norm_grad_op(dy, x, gd, mean, rstd, data_format=fmt, epsilon=EPS)
    assert dx.shape == x.shape and dg.shape == (C,) and db.shape == (C,)
    torch.cuda.synchronize()
    flat = (N, C, D) if cf else (N, D, C)
    x64, dy64 = _np(x).reshape(flat), _np(dy).reshape(flat)
    y_ref, m_ref, r_ref = O.in_fwd_np(x64, gamma, beta, EPS, cf)
    dx_ref, dg_ref, db_ref = O.in_bwd_np(dy64, x64, gamma, _np(mean), _np(rstd), cf)
    tol = TOL[dtype]
    assert_close(_np(y).reshape(flat), y_ref, tol["y"], "y")
    assert_close(_np(mean), m_ref, tol["stat"], "mean")
    assert_close(_np(rstd), r_ref, tol["stat"], "inv_std")
    assert_close(_np(dx).reshape(flat), dx_ref, tol["dx"], "dx")
    assert_close(_np(dg), dg_ref, tol["dw"], "dgamma")
    assert_close(_np(db), db_ref, tol["dw"], "dbeta")


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("shape,axis", [((4, 8, 16), [1, 2]), ((4, 8, 16), -1), ((12, 4, 8, 8), [1, 2, 3]),
                                        ((3, 1000), [-1]), ((64, 1024), [1])])
def test_layer_normalization_layer(shape, axis, dtype):
    """The layer against torch.nn.functional.layer_norm in float32 on the same device, with
    autograd through both (the reference compares against the Keras layer the same way,
    fused_layer_norm_test.py:102-135)."""
    import torch
    import torch.nn.functional as F

    from atex_amd import nv_norms

    print(f"layer LN shape={shape} axis={axis} dtype={dtype}", flush=True)
    x, rng = _rand(shape, dtype, 60)
    dy, _ = _rand(shape, dtype, 61)
    layer = nv_norms.LayerNormalization(axis=axis, epsilon=EPS)
    layer.build(shape, device="cuda")
    ax = [axis] if isinstance(axis, int) else list(axis)
    wshape = tuple(shape[a] for a in ax)
    gamma = rng.uniform(0.5, 1.5, size=wshape).astype(np.float32)
    beta = (rng.standard_normal(wshape) * 0.1).astype(np.float32)
    layer.set_weights([gamma, beta])
    xin = x.clone().requires_grad_(True)
    y = layer(xin)
    assert y.dtype == x.dtype and y.shape == x.shape
    y.backward(dy)

    xr = x.float().clone().requires_grad_(True)
    gr = torch.from_numpy(gamma).cuda().requires_grad_(True)
    br = torch.from_numpy(beta).cuda().requires_grad_(True)
    yr = F.layer_norm(xr, wshape, gr, br, EPS)
    yr.backward(dy.float())
    torch.cuda.synchronize()
    tol = TOL[dtype]
    assert_close(_np(y), _np(yr), tol["y"], "y")
    assert_close(_np(xin.grad), _np(xr.grad), tol["dx"], "dx")
    assert layer.gamma.grad.shape == layer.gamma.shape
    assert_close(_np(layer.gamma.grad), _np(gr.grad), max(tol["dw"], 2e-5), "dgamma")
    assert_close(_np(layer.beta.grad), _np(br.grad), max(tol["dw"], 2e-5), "dbeta")


@pytest.mark.parametrize("dtype", ["f32", "f16"])
@pytest.mark.parametrize("shape,axis", [((2, 16, 16, 32), -1), ((2, 32, 16, 16), 1), ((2, 6, 8, 10, 16), -1),
                                        ((2, 16, 6, 8, 10), 1), ((3, 5, 7, 9), 1), ((3, 7, 9, 5), -1)])
def test_instance_normalization_layer(shape, axis, dtype):
    """Against torch's group_norm with one group per channel in float32 (channels-last
    inputs are permuted for it), autograd through both."""
    import torch
    import torch.nn.functional as F

    from atex_amd import nv_norms

    print(f"layer IN shape={shape} axis={axis} dtype={dtype}", flush=True)
    x, rng = _rand(shape, dtype, 70)
    dy, _ = _rand(shape, dtype, 71)
    C = shape[axis]
    layer = nv_norms.InstanceNormalization(axis=axis, epsilon=EPS)
    layer.build(shape, device="cuda")
    gamma, beta = util.affine_params(rng, C)
    layer.set_weights([gamma, beta])
    xin = x.clone().requires_grad_(True)
    y = layer(xin)
    y.backward(dy)

    nd = len(shape)
    to_cf = (0, nd - 1) + tuple(range(1, nd - 1))
    to_cl = (0,) + tuple(range(2, nd)) + (1,)
    xr = x.float().clone().requires_grad_(True)
    gr = torch.from_numpy(gamma).cuda().requires_grad_(True)
    br = torch.from_numpy(beta).cuda().requires_grad_(True)
    xcf = xr if axis == 1 else xr.permute(to_cf)
    yr = F.group_norm(xcf, C, gr, br, EPS)
    if axis != 1:
        yr = yr.permute(to_cl)
    yr.backward(dy.float())
    torch.cuda.synchronize()
    tol = TOL[dtype]
    assert_close(_np(y), _np(yr), tol["y"], "y")
    assert_close(_np(xin.grad), _np(xr.grad), tol["dx"], "dx")
    assert_close(_np(layer.gamma.grad), _np(gr.grad), max(tol["dw"], 2e-5), "dgamma")
    assert_close(_np(layer.beta.grad), _np(br.grad), max(tol["dw"], 2e-5), "dbeta")


def test_layer_mixed_precision_weights_stay_float32():
    """Weights and their gradients are float32 whatever the activation dtype
    (fused_layer_norm_test.py:262-289 runs the layer under a mixed_float16 policy)."""
    import torch

    from atex_amd import nv_norms

    x = torch.randn(8, 64, device="cuda", dtype=torch.float16, requires_grad=True)
    layer = nv_norms.LayerNormalization(axis=-1)
    y = layer(x)
    y.float().sum().backward()
    assert y.dtype == torch.float16 and x.grad.dtype == torch.float16
    assert layer.gamma.dtype == torch.float32 and layer.gamma.grad.dtype == torch.float32
    assert layer.get_config() == {"axis": [1], "epsilon": 1e-3}


def test_gradient_registration():
    """The registered gradient functions take the forward op's inputs / outputs and the
    upstream gradients and return (dx, dscale, doffset) (nv_norm_ops.py:27-66)."""
    import torch

    from atex_amd import nv_norms
    from atex_amd.nv_norms.layers import _OpRecord

    x = torch.randn(4, 6, 8, device="cuda")
    g = torch.rand(48, device="cuda") + 0.5
    b = torch.zeros(48, device="cuda")
    y, m, r = nv_norms.fused_layer_norm_op(x, g, b, axis=[1, 2])
    op = _OpRecord([x, g, b], [y, m, r], {"axis": [1, 2], "epsilon": 0.001})
    dy = torch.randn_like(x)
    dx, dg, db = nv_norms._layer_norm_grad(op, dy, None, None)
    dx2, dg2, db2 = nv_norms.fused_layer_norm_grad_op(dy, x, g, m, r, axis=[1, 2])
    torch.cuda.synchronize()
    assert torch.equal(dx, dx2) and torch.equal(dg, dg2) and torch.equal(db, db2)
