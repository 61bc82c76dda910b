"""The library's two kernel sets against each other: the same op on the same inputs placed on
the GPU (HIP kernels) and in host memory (CPU kernels), through the op-level Python surface.
Both compute in float32 from the same rounded inputs, so they agree to float32 rounding in the
statistics and the parameter gradients, and to one unit in the last place of the storage type
in y and dx."""
import numpy as np
import pytest

from tests import util

pytestmark = pytest.mark.gpu

EPS = 1e-3


def _ulp_close(a, b, dtype, frac_exact=0.98):
    """a, b: torch tensors of the storage dtype; equal up to one storage ulp, and mostly equal."""
    import torch

    af, bf = a.float(), b.float()
    if dtype == "f32":
        assert torch.allclose(af, bf, rtol=2e-5, atol=2e-6)
        return
    ulp = torch.finfo(a.dtype).eps * torch.maximum(af.abs(), bf.abs()).clamp_min(torch.finfo(a.dtype).tiny)
    assert bool(((af - bf).abs() <= ulp * 1.01 + 1e-6).all())
    assert float((af == bf).float().mean()) >= frac_exact


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("shape,axis", [((64, 1024), [-1]), ((6, 5, 96), [1, 2]), ((3, 40000), [-1])])
def test_layer_norm_gpu_vs_cpu(shape, axis, dtype):
    import torch

    from atex_amd import nv_norms

    tdt = util.torch_dtype(dtype)
    g = torch.Generator().manual_seed(60)
    x = (torch.randn(shape, generator=g) + 1.5).to(tdt)
    dy = torch.randn(shape, generator=g).to(tdt)
    wshape = tuple(shape[a] for a in sorted(a % len(shape) for a in axis))
    gamma = torch.rand(wshape, generator=g) + 0.5
    beta = torch.randn(wshape, generator=g) * 0.1
    print(f"LN gpu vs cpu shape={shape} axis={axis} dtype={dtype}", flush=True)
    yc, mc, rc = nv_norms.fused_layer_norm_op(x, gamma, beta, axis=axis, epsilon=EPS)
    dxc, dgc, dbc = nv_norms.fused_layer_norm_grad_op(dy, x, gamma, mc, rc, axis=axis)
    yg, mg, rg = nv_norms.fused_layer_norm_op(x.cuda(), gamma.cuda(), beta.cuda(), axis=axis, epsilon=EPS)
    dxg, dgg, dbg = nv_norms.fused_layer_norm_grad_op(dy.cuda(), x.cuda(), gamma.cuda(), mc.cuda(), rc.cuda(), axis=axis)
    torch.cuda.synchronize()
    assert torch.allclose(mg.cpu(), mc, rtol=1e-5, atol=1e-6)
    assert torch.allclose(rg.cpu(), rc, rtol=1e-5, atol=1e-6)
    _ulp_close(yg.cpu(), yc, dtype)
    _ulp_close(dxg.cpu(), dxc, dtype, frac_exact=0.95)
    n_rows = x.numel() // gamma.numel()
    assert torch.allclose(dgg.cpu(), dgc, rtol=1e-4, atol=1e-5 * n_rows ** 0.5)
    assert torch.allclose(dbg.cpu(), dbc, rtol=1e-4, atol=1e-5 * n_rows ** 0.5)


@pytest.mark.parametrize("dtype", ["f32", "f16"])
@pytest.mark.parametrize("fmt,shape", [("NHWC", (4, 24, 24, 32)), ("NCHW", (4, 32, 24, 24)), ("NDHWC", (2, 6, 7, 8, 10)),
                                       ("NCDHW", (2, 10, 6, 7, 8))])
def test_instance_norm_gpu_vs_cpu(fmt, shape, dtype):
    import torch

    from atex_amd import nv_norms

    tdt = util.torch_dtype(dtype)
    g = torch.Generator().manual_seed(61)
    C = shape[1] if fmt[1] == "C" else shape[-1]
    x = (torch.randn(shape, generator=g) - 0.7).to(tdt)
    dy = torch.randn(shape, generator=g).to(tdt)
    gamma = torch.rand(C, generator=g) + 0.5
    beta = torch.randn(C, generator=g) * 0.1
    print(f"IN gpu vs cpu {fmt} shape={shape} dtype={dtype}", flush=True)
    yc, mc, rc = nv_norms.fused_instance_norm_op(x, gamma, beta, data_format=fmt, epsilon=EPS)
    dxc, dgc, dbc = nv_norms.fused_instance_norm_grad_op(dy, x, gamma, mc, rc, data_format=fmt)
    yg, mg, rg = nv_norms.fused_instance_norm_op(x.cuda(), gamma.cuda(), beta.cuda(), data_format=fmt, epsilon=EPS)
    dxg, dgg, dbg = nv_norms.fused_instance_norm_grad_op(dy.cuda(), x.cuda(), gamma.cuda(), mc.cuda(), rc.cuda(),
                                                         data_format=fmt)
    torch.cuda.synchronize()
    assert torch.allclose(mg.cpu(), mc, rtol=1e-5, atol=1e-6)
    assert torch.allclose(rg.cpu(), rc, rtol=1e-5, atol=1e-6)
    _ulp_close(yg.cpu(), yc, dtype)
    _ulp_close(dxg.cpu(), dxc, dtype, frac_exact=0.95)
    n_terms = x.numel() // C
    assert torch.allclose(dgg.cpu(), dgc, rtol=1e-4, atol=1e-5 * n_terms ** 0.5)
    assert torch.allclose(dbg.cpu(), dbc, rtol=1e-4, atol=1e-5 * n_terms ** 0.5)
