"""A NaN or Inf in one row / one (instance, channel) plane stays there: every other row's y, dx,
mean and inv_std are bit-identical to the clean run (the masked lanes and clamped duplicate
loads of the kernels must select, never multiply by zero), and the poisoned row is non-finite.
dgamma / dbeta sum over rows, so for LayerNorm only the poisoned COLUMNS of dgamma may differ
... except that x-hat of the poisoned row is NaN everywhere, which makes every column NaN: only
the channel-wise InstanceNorm gradients of OTHER channels are required to stay clean."""
import numpy as np
import pytest

from tests import util

pytestmark = pytest.mark.gpu

EPS = 1e-3


def _rows_equal(a, b, keep):
    import torch

    return torch.equal(a[keep], b[keep])


@pytest.mark.parametrize("bad", [float("nan"), float("inf")])
@pytest.mark.parametrize("N,D,row,col", [
    (37, 1000, 36, 999),     # ragged lane groups, last element of the last row
    (37, 1000, 0, 0),
    (5000, 10, 4999, 9),     # one thread per row
    (5000, 10, 17, 3),
    (33, 4096, 32, 5),       # wave groups (backward)
    (9, 12288, 4, 12287),    # one workgroup per row
    (5, 70001, 2, 70000),    # 2-D tiles, the ragged tail element
    (5, 70001, 4, 8191),
])
def test_layer_norm_row_isolation(N, D, row, col, bad):
    import torch

    capi = util.Capi()
    g = torch.Generator(device="cuda")
    g.manual_seed(3)
    x = torch.randn((N, D), device="cuda", generator=g).half()
    dy = torch.randn((N, D), device="cuda", generator=g).half()
    gamma = torch.rand(D, device="cuda", generator=g) + 0.5
    beta = torch.randn(D, device="cuda", generator=g) * 0.1
    print(f"LN non-finite isolation N={N} D={D} at ({row},{col}) value {bad}", flush=True)
    y0, m0, r0 = capi.ln_fwd(x, gamma, beta, EPS, "f16")
    dx0, _, _ = capi.ln_bwd(dy, x, gamma, m0, r0, "f16")
    xb = x.clone()
    xb[row, col] = bad
    y1, m1, r1 = capi.ln_fwd(xb, gamma, beta, EPS, "f16")
    dx1, _, _ = capi.ln_bwd(dy, xb, gamma, m1, r1, "f16")
    torch.cuda.synchronize()
    keep = torch.ones(N, dtype=torch.bool, device="cuda")
    keep[row] = False
    for a, b, name in ((y0, y1, "y"), (m0, m1, "mean"), (r0, r1, "inv_std"), (dx0, dx1, "dx")):
        assert _rows_equal(a, b, keep), name
    assert not torch.isfinite(m1[row]) and not torch.isfinite(y1[row].float()).all()
    assert not torch.isfinite(dx1[row].float()).all()


@pytest.mark.parametrize("bad", [float("nan"), float("inf")])
@pytest.mark.parametrize("channel_first", [False, True])
@pytest.mark.parametrize("N,C,S,n,c,s", [
    (3, 16, 1000, 2, 15, 999),      # resident / small slabs
    (3, 20, 1000, 1, 19, 0),        # ragged channel count
    (2, 8, 300001, 1, 3, 300000),   # streamed slabs / split planes, last pixel (a pivot sample)
    (2, 8, 300001, 0, 7, 150000),   # the middle pivot sample
    (50, 3, 17, 49, 2, 16),         # fewer channels than a vector
])
def test_instance_norm_plane_isolation(N, C, S, n, c, s, channel_first, bad):
    import torch

    capi = util.Capi()
    g = torch.Generator(device="cuda")
    g.manual_seed(4)
    shape = (N, C, S) if channel_first else (N, S, C)
    x = torch.randn(shape, device="cuda", generator=g).half()
    dy = torch.randn(shape, device="cuda", generator=g).half()
    gamma = torch.rand(C, device="cuda", generator=g) + 0.5
    beta = torch.randn(C, device="cuda", generator=g) * 0.1
    print(f"IN non-finite isolation N={N} C={C} S={S} channel_first={channel_first} at "
          f"({n},{c},{s}) value {bad}", flush=True)
    y0, m0, r0 = capi.in_fwd(x, gamma, beta, EPS, "f16", channel_first)
    dx0, dg0, db0 = capi.in_bwd(dy, x, gamma, m0, r0, "f16", channel_first)
    xb = x.clone()
    if channel_first:
        xb[n, c, s] = bad
    else:
        xb[n, s, c] = bad
    y1, m1, r1 = capi.in_fwd(xb, gamma, beta, EPS, "f16", channel_first)
    dx1, dg1, db1 = capi.in_bwd(dy, xb, gamma, m1, r1, "f16", channel_first)
    torch.cuda.synchronize()
    keep = torch.ones((N, C), dtype=torch.bool, device="cuda")
    keep[n, c] = False
    assert torch.equal(m0[keep], m1[keep]) and torch.equal(r0[keep], r1[keep])
    assert not torch.isfinite(m1[n, c])

    def planes(t):  # [N, C, S] view of either layout
        return t if channel_first else t.permute(0, 2, 1)

    for a, b, name in ((y0, y1, "y"), (dx0, dx1, "dx")):
        assert torch.equal(planes(a)[keep], planes(b)[keep]), name
        assert not torch.isfinite(planes(b)[n, c].float()).all(), name
    other = torch.ones(C, dtype=torch.bool, device="cuda")
    other[c] = False
    assert torch.equal(dg0[other], dg1[other]) and torch.equal(db0[other], db1[other])
    assert not torch.isfinite(dg1[c])
