"""bench.py times the dominant backward kernel alone through the benchmark build of the
library (libatex_norms_hip_bench.so: the product sources compiled with -DATEXN_BENCH_BUILD,
which adds the launch-planning switches).  With every switch at its default that build must be
the product library in all but name: the same plans (workspace sizes) and bit-identical outputs
on the shapes the benchmark quotes, so that a duration measured on one holds for the other.
"""
import numpy as np
import pytest

from tests import util

pytestmark = pytest.mark.gpu

EPS = 1e-3

# (op, dtype, dims): the two target shapes in both layouts, the hidden-size sweep at reduced row
# counts that keep each shape on its full-size kernel family, and a long-row / staged case
SHAPES = [
    ("ln", "f16", (8192, 1024)),
    ("ln", "f32", (32, 1024)),
    ("ln", "bf16", (4096, 128)),
    ("ln", "f16", (2048, 4096)),
    ("ln", "f16", (2048, 12288)),
    ("ln", "f16", (512, 18432)),
    ("ln", "f16", (8, 70001)),
    ("in", "f16", (8, 64, 16384, False)),
    ("in", "f16", (8, 64, 16384, True)),
    ("in", "f16", (2, 32, 262144, False)),
    ("in", "f16", (2, 32, 262144, True)),
    ("in", "f16", (8, 64, 36864, True)),
]


def _bits_equal(a, b):
    import torch

    return torch.equal(a.view(torch.uint8), b.view(torch.uint8))


@pytest.mark.parametrize("op,dtype,dims", SHAPES)
def test_bench_build_is_bit_identical_to_product(op, dtype, dims):
    import torch

    from oracle import oracle as O

    product, bench = util.Capi(), util.Capi(bench=True)
    assert product.L is not bench.L
    assert bench.L.atexn_set_tuning(b"bwd_stage_mask", 3) == 0
    code = O.DTYPE_CODE[dtype]
    print(f"bench build vs product op={op} dtype={dtype} dims={dims}", flush=True)
    if op == "ln":
        N, D = dims
        for q in ("atexn_layer_norm_fwd_workspace_bytes", "atexn_layer_norm_bwd_workspace_bytes"):
            assert getattr(product.L, q)(code, N, D) == getattr(bench.L, q)(code, N, D), q
        x, gamma, beta, dy = util.ln_inputs("row_mean", N, D, dtype, 60)
        run = lambda c, xd, dyd, gd, bd: (lambda f: f + c.ln_bwd(dyd, xd, gd, f[1], f[2], dtype))(  # noqa: E731
            c.ln_fwd(xd, gd, bd, EPS, dtype))
    else:
        N, C, S, cf = dims
        for q in ("atexn_instance_norm_fwd_workspace_bytes", "atexn_instance_norm_bwd_workspace_bytes"):
            assert getattr(product.L, q)(code, 0 if cf else 1, N, C, S) == getattr(bench.L, q)(code, 0 if cf else 1, N, C, S), q
        x, gamma, beta, dy = util.in_inputs(N, C, S, dtype, cf, 61)
        run = lambda c, xd, dyd, gd, bd: (lambda f: f + c.in_bwd(dyd, xd, gd, f[1], f[2], dtype, cf))(  # noqa: E731
            c.in_fwd(xd, gd, bd, EPS, dtype, cf))
    xd, dyd = util.to_device(x, dtype), util.to_device(dy, dtype)
    gd, bd = torch.from_numpy(gamma).cuda(), torch.from_numpy(beta).cuda()
    a = run(product, xd, dyd, gd, bd)
    b = run(bench, xd, dyd, gd, bd)
    torch.cuda.synchronize()
    for name, u, v in zip(("y", "mean", "inv_std", "dx", "dgamma", "dbeta"), a, b):
        assert _bits_equal(u, v), f"{name}: the benchmark build differs from the product library"
