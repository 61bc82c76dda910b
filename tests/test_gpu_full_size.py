"""Benchmark configurations 2 and 4 at their full sizes.

Configuration 2 (LayerNorm hidden-size sweep, [262144, 128], [16384, 4096], [2048, 12288] in
fp16 and bf16) runs through the kernel-level entry points against the oracle's float64
flavour on every element: the launch plan depends on the row count (rows per lane group,
block size, grid), so the instantiations that run at the full row counts are not the ones a
reduced row count selects.

Configuration 4, x fp16 [2, 128, 128, 128, 32] (both layouts), runs through the op-level
entry points.  The oracle still runs in a few seconds on the box's
cores for one forward + backward, so the values are compared directly; on top of that come
the size-independent properties the statistics must satisfy whatever the size:

* per (n, c): mean(y - beta) = 0 and mean(((y - beta) / gamma)^2) = var / (var + eps);
* per (n, c): sum(dx) = 0 and sum(dx * (x - mean)) = 0 (dx is orthogonal to 1 and to x - mean);
* dbeta = sum(dy), dgamma = sum(dy * xhat) recomputed from the returned statistics;
* the two layouts give the same statistics and weight gradients for transposed inputs.

Configurations 0 and 1 run at full size in test_gpu_layer_norm.py, configuration 3 in
test_gpu_instance_norm.py.
"""
import numpy as np
import pytest

from tests import util
from tests.util import TOL, assert_close

pytestmark = pytest.mark.gpu

EPS = 1e-3
N, C, SP = 2, 32, (128, 128, 128)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("rows,D", [(262144, 128), (16384, 4096), (2048, 12288)])
def test_config2_full_row_counts(coracle, rows, D, dtype):
    from tests.test_gpu_layer_norm import run_case

    run_case(util.Capi(), coracle, "scaled_rows", rows, D, dtype, 2)


@pytest.fixture(scope="module")
def volume():
    """Generated on the device (134M elements per tensor): deterministic from the seed."""
    import torch

    g = torch.Generator(device="cuda").manual_seed(1004)
    x = torch.randn((N, *SP, C), generator=g, device="cuda", dtype=torch.float32)
    x += torch.rand((1, 1, 1, 1, C), generator=g, device="cuda") * 2 - 1
    dy = torch.randn((N, *SP, C), generator=g, device="cuda", dtype=torch.float32)
    gamma = torch.rand(C, generator=g, device="cuda") + 0.5
    beta = torch.randn(C, generator=g, device="cuda") * 0.1
    return x.half(), dy.half(), gamma, beta


def _properties(x, dy, y, mean, rstd, dx, dg, db, gamma, beta, red, bshape):
    """All arguments are device tensors; reductions in float64 on the device."""
    import torch

    D = float(np.prod(SP))
    m = mean.double().reshape(bshape)
    r = rstd.double().reshape(bshape)
    cshape = [1] * len(bshape)
    cshape[bshape.index(C)] = C
    g = gamma.double().reshape(cshape)
    b = beta.double().reshape(cshape)
    xh = (x.double() - m) * r
    # forward
    z = (y.double() - b) / g
    assert float(z.mean(dim=red).abs().max()) < 2e-4          # fp16 rounding of y averages out
    var_ratio = (z * z).mean(dim=red)
    expect = 1.0 - EPS * (rstd.double() ** 2)                  # var / (var + eps)
    assert_close(var_ratio.cpu().numpy(), expect.cpu().numpy(), 1e-3, "mean(xhat^2)")
    del z
    # backward
    dyd = dy.double()
    db_ref = dyd.sum(dim=red).sum(dim=0)
    dg_ref = (dyd * xh).sum(dim=red).sum(dim=0)
    assert_close(db.cpu().numpy(), db_ref.cpu().numpy(), 1e-3, "dbeta")
    assert_close(dg.cpu().numpy(), dg_ref.cpu().numpy(), 1e-3, "dgamma")
    dxd = dx.double()
    s0 = dxd.sum(dim=red) / D
    s1 = (dxd * xh).sum(dim=red) / D
    # each dx element carries an fp16 rounding error of relative size 2^-11; the sums of D of
    # them average to well under 1e-4 of a typical |dx| (about rstd * gamma, order 1)
    assert float(s0.abs().max()) < 1e-4, float(s0.abs().max())
    assert float(s1.abs().max()) < 1e-4, float(s1.abs().max())


@pytest.mark.parametrize("channel_first", [False, True])
def test_config4_full_volume(volume, coracle, channel_first):
    import torch

    from atex_amd import nv_norms

    x, dy, gamma, beta = volume
    fmt = "NCDHW" if channel_first else "NDHWC"
    print(f"config4 full {fmt} x{tuple(x.shape)} fp16", flush=True)
    if channel_first:
        x = x.permute(0, 4, 1, 2, 3).contiguous()
        dy = dy.permute(0, 4, 1, 2, 3).contiguous()
    y, mean, rstd = nv_norms.fused_instance_norm_op(x, gamma, beta, data_format=fmt, epsilon=EPS)
    dx, dg, db = nv_norms.fused_instance_norm_grad_op(dy, x, gamma, mean, rstd, data_format=fmt)
    torch.cuda.synchronize()
    red = (2, 3, 4) if channel_first else (1, 2, 3)
    bshape = [N, C, 1, 1, 1] if channel_first else [N, 1, 1, 1, C]
    _properties(x, dy, y, mean, rstd, dx, dg, db, gamma, beta, red, bshape)

    # direct comparison with the oracle
    D = int(np.prod(SP))
    flat = (N, C, D) if channel_first else (N, D, C)
    xh, dyh = x.cpu().numpy().reshape(flat), dy.cpu().numpy().reshape(flat)
    gh, bh = gamma.cpu().numpy(), beta.cpu().numpy()
    y_ref, m_ref, r_ref = coracle.in_fwd(xh, gh, bh, EPS, "f16", channel_first)
    tol = TOL["f16"]
    assert_close(util.to_host(mean), m_ref, tol["stat"], "mean")
    assert_close(util.to_host(rstd), r_ref, tol["stat"], "inv_std")
    assert_close(y.cpu().numpy().reshape(flat), y_ref, tol["y"], "y")
    del y_ref
    dx_ref, dg_ref, db_ref = coracle.in_bwd(dyh, xh, gh, util.to_host(mean), util.to_host(rstd), "f16", channel_first)
    assert_close(dx.cpu().numpy().reshape(flat), dx_ref, tol["dx"], "dx")
    assert_close(util.to_host(dg), dg_ref, tol["dw"], "dgamma")
    assert_close(util.to_host(db), db_ref, tol["dw"], "dbeta")


def test_config4_layouts_agree(volume):
    import torch

    from atex_amd import nv_norms

    x, dy, gamma, beta = volume
    y1, m1, r1 = nv_norms.fused_instance_norm_op(x, gamma, beta, data_format="NDHWC", epsilon=EPS)
    _, dg1, db1 = nv_norms.fused_instance_norm_grad_op(dy, x, gamma, m1, r1, data_format="NDHWC")
    xc = x.permute(0, 4, 1, 2, 3).contiguous()
    dyc = dy.permute(0, 4, 1, 2, 3).contiguous()
    y2, m2, r2 = nv_norms.fused_instance_norm_op(xc, gamma, beta, data_format="NCDHW", epsilon=EPS)
    _, dg2, db2 = nv_norms.fused_instance_norm_grad_op(dyc, xc, gamma, m2, r2, data_format="NCDHW")
    torch.cuda.synchronize()
    assert_close(util.to_host(m2), util.to_host(m1), 1e-5, "mean")
    assert_close(util.to_host(r2), util.to_host(r1), 1e-5, "inv_std")
    assert_close(util.to_host(dg2), util.to_host(dg1), 1e-4, "dgamma")
    assert_close(util.to_host(db2), util.to_host(db1), 1e-4, "dbeta")
    # y differs by at most one fp16 ulp where the two float32 results straddle a rounding boundary
    diff = (y2.permute(0, 2, 3, 4, 1).float() - y1.float()).abs()
    assert float(diff.max()) <= 2.0 ** -8 * 1.01 and float((diff > 0).float().mean()) < 1e-2
