"""Inputs with a large common offset (|mean| / std = 10 ... 1000) through every kernel family.
In float32 the input's own rounding is 6e-8 * |mean|, so no float32 evaluation can do better
than about 1e-7 * |mean| / std in y; the bound checked here is that floor times a small
constant, i.e. the statistics (exact two-pass over registers, or sums around a pivot taken
from the data) lose nothing beyond what the representation already lost.  A formulation
around zero (sum x^2 - mean^2) would fail these by orders of magnitude."""
import numpy as np
import pytest

from tests import util
from tests.util import assert_close

pytestmark = pytest.mark.gpu

EPS = 1e-3


def _err_bounds(kappa):
    floor = 6e-8 * kappa              # relative to std = 1
    return dict(mean=1e-6, y=1e-5 + 40 * floor, rstd=1e-5 + 40 * floor)


@pytest.mark.parametrize("kappa", [10.0, 100.0, 1000.0])
@pytest.mark.parametrize("N,D", [(300, 1024), (50, 1000), (5000, 10), (16, 12288), (4, 70001)])
def test_layer_norm_offset(coracle, N, D, kappa):
    import torch

    capi = util.Capi()
    rng = util.rng_for(300)
    x = (rng.standard_normal((N, D)) + kappa * rng.choice([-1.0, 1.0], size=(N, 1))).astype(np.float32)
    gamma, beta = util.affine_params(rng, D)
    print(f"LN offset kappa={kappa} N={N} D={D}", flush=True)
    y_ref, m_ref, r_ref = coracle.ln_fwd(x, gamma, beta, EPS, "f32")
    y, m, r = capi.ln_fwd(torch.from_numpy(x).cuda(), torch.from_numpy(gamma).cuda(),
                          torch.from_numpy(beta).cuda(), EPS, "f32")
    torch.cuda.synchronize()
    b = _err_bounds(kappa)
    assert np.max(np.abs(util.to_host(m) - m_ref) / np.abs(m_ref)) <= b["mean"]
    assert np.max(np.abs(util.to_host(r) - r_ref) / r_ref) <= b["rstd"]
    assert np.max(np.abs(util.to_host(y) - y_ref)) <= b["y"] * 2.0  # |gamma| <= 1.5, |xhat| <~ 5


@pytest.mark.parametrize("kappa", [10.0, 100.0, 1000.0])
@pytest.mark.parametrize("channel_first", [False, True])
@pytest.mark.parametrize("N,C,S", [(4, 32, 4096), (2, 16, 300000), (1, 8, 33), (600, 8, 20)])
def test_instance_norm_offset(coracle, N, C, S, channel_first, kappa):
    import torch

    capi = util.Capi()
    rng = util.rng_for(301)
    x = rng.standard_normal((N, S, C)) + kappa * rng.choice([-1.0, 1.0], size=(N, 1, C))
    x = x.astype(np.float32)
    if channel_first:
        x = np.ascontiguousarray(np.transpose(x, (0, 2, 1)))
    gamma, beta = util.affine_params(rng, C)
    print(f"IN offset kappa={kappa} N={N} C={C} spatial={S} channel_first={channel_first}", flush=True)
    y_ref, m_ref, r_ref = coracle.in_fwd(x, gamma, beta, EPS, "f32", channel_first)
    y, m, r = capi.in_fwd(torch.from_numpy(x).cuda(), torch.from_numpy(gamma).cuda(),
                          torch.from_numpy(beta).cuda(), EPS, "f32", channel_first)
    torch.cuda.synchronize()
    b = _err_bounds(kappa)
    assert np.max(np.abs(util.to_host(m) - m_ref) / np.abs(m_ref)) <= b["mean"]
    assert np.max(np.abs(util.to_host(r) - r_ref) / r_ref) <= b["rstd"]
    assert np.max(np.abs(util.to_host(y) - y_ref)) <= b["y"] * 2.0


# Kernel families whose statistics stream through the data (everything that is not an exact
# two-pass over a register-resident row): name -> (layout, N, C, D).  "cl" = channels-last.
OUTLIER_CASES = {
    "channels-last, register slabs, 64 slabs merged by stage 2": ("cl", 8, 64, 16384),
    "channels-last, streaming slabs merged by stage 2": ("cl", 8, 32, 1 << 17),
    "channels-last, register slabs, merge launch": ("cl", 1, 8, 1 << 19),
    "channels-last, streaming slabs, merge launch": ("cl", 1, 32, 1 << 19),
    "channels-last, C not a multiple of the vector": ("cl", 16, 6, 5000),
    "channels-last, C not a multiple of the vector, merge launch": ("cl", 2, 6, 50000),
    "channels-last, single pass": ("cl", 512, 32, 256),
    "channel-first, planes split over workgroups": ("cf", 1, 3, 1 << 19),
    "LayerNorm tiles (rows too long for registers)": ("ln", 6, 1, 70001),
}


@pytest.mark.parametrize("kappa", [100.0, 1000.0])
@pytest.mark.parametrize("case", sorted(OUTLIER_CASES))
def test_outlier_samples(coracle, case, kappa):
    """The bulk of every instance / row is N(kappa, 1) while the places a kernel could take a
    pivot or a first sample from are 0, i.e. kappa standard deviations away: the first, middle
    and last pixel of an instance (an image with zero-padded corners), and the first element of
    the first few threads' shares of a row.  Statistics must keep the float32 tolerance: the
    reference's Welford pushes do (norm_util.h:182-211)."""
    import torch

    layout, N, C, D = OUTLIER_CASES[case]
    capi = util.Capi()
    rng = util.rng_for(302)
    print(f"outlier samples: {case} kappa={kappa} N={N} C={C} D={D}", flush=True)
    if layout == "ln":
        x = (rng.standard_normal((N, D)) + kappa).astype(np.float32)
        x[:, [0, 4, 8, 12, D // 2, D - 1]] = 0
        gamma, beta = util.affine_params(rng, D)
        y_ref, m_ref, r_ref = coracle.ln_fwd(x, gamma, beta, EPS, "f32")
        y, m, r = capi.ln_fwd(torch.from_numpy(x).cuda(), torch.from_numpy(gamma).cuda(),
                              torch.from_numpy(beta).cuda(), EPS, "f32")
    else:
        x = (rng.standard_normal((N, D, C)) + kappa).astype(np.float32)
        x[:, [0, 1, 2, 3, D // 2, D - 1], :] = 0
        cf = layout == "cf"
        if cf:
            x = np.ascontiguousarray(np.transpose(x, (0, 2, 1)))
            x[:, :, [4, 8, 12]] = 0
        gamma, beta = util.affine_params(rng, C)
        y_ref, m_ref, r_ref = coracle.in_fwd(x, gamma, beta, EPS, "f32", cf)
        y, m, r = capi.in_fwd(torch.from_numpy(x).cuda(), torch.from_numpy(gamma).cuda(),
                              torch.from_numpy(beta).cuda(), EPS, "f32", cf)
    torch.cuda.synchronize()
    tol = util.TOL["f32"]["stat"]
    assert_close(util.to_host(m), m_ref, tol, "mean")
    assert_close(util.to_host(r), r_ref, tol, "inv_std")
    # y = (x - mean) * r: x - mean carries the float32 rounding of mean, 6e-8 * kappa
    assert np.max(np.abs(util.to_host(y) - y_ref) / (1.0 + np.abs(y_ref))) <= 1e-5 + 40 * 6e-8 * kappa


def test_constant_rows_and_extremes():
    """Constant rows give y = beta and inv_std = eps^-1/2 exactly where the kernel centres
    exactly; fp16 rows at the top of the fp16 range do not overflow (statistics are float32)."""
    import torch

    capi = util.Capi()
    for D in (10, 1024, 5000, 70000):
        x = torch.full((8, D), 3.25, device="cuda", dtype=torch.float32)
        g = torch.full((D,), 1.5, device="cuda")
        b = torch.full((D,), -0.5, device="cuda")
        y, m, r = capi.ln_fwd(x, g, b, EPS, "f32")
        torch.cuda.synchronize()
        assert torch.allclose(m, torch.full_like(m, 3.25), rtol=1e-6)
        assert torch.allclose(r, torch.full_like(r, EPS ** -0.5), rtol=1e-5)
        assert torch.allclose(y, torch.full_like(y, -0.5), atol=2e-4), (D, float((y + 0.5).abs().max()))
    big = torch.empty((16, 2048), device="cuda", dtype=torch.float16).uniform_(-1, 1) * 60000
    y, m, r = capi.ln_fwd(big, torch.ones(2048, device="cuda"), torch.zeros(2048, device="cuda"), EPS, "f16")
    torch.cuda.synchronize()
    assert torch.isfinite(y.float()).all() and torch.isfinite(m).all() and torch.isfinite(r).all()
    assert float(y.float().abs().max()) < 4.0
