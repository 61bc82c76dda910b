"""The HIP path against the committed golden fixtures (torch CPU float64 + autograd, see
tests/golden/make_golden.py), with no oracle in between: kernel-level C ABI, tolerances
of the acceptance bar."""
import glob
import os

import numpy as np
import pytest

from tests import util
from tests.util import TOL, assert_close

pytestmark = pytest.mark.gpu

GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "*.npz")))


@pytest.fixture(scope="module")
def capi():
    return util.Capi()


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p)[:-4] for p in GOLDEN])
def test_hip_matches_golden(capi, path):
    import torch

    g = np.load(path)
    dtype, eps, kind = str(g["dtype"]), float(g["eps"]), str(g["kind"])
    print(f"golden {os.path.basename(path)} kind={kind} dtype={dtype} x{g['x'].shape}", flush=True)
    tol = TOL[dtype]
    xd, dyd = util.to_device(g["x"], dtype), util.to_device(g["dy"], dtype)
    gd, bd = torch.from_numpy(g["gamma"]).cuda(), torch.from_numpy(g["beta"]).cuda()
    mean32 = torch.from_numpy(g["mean"].astype(np.float32)).cuda()
    rstd32 = torch.from_numpy(g["inv_std"].astype(np.float32)).cuda()
    if kind == "ln":
        y, m, r = capi.ln_fwd(xd, gd, bd, eps, dtype)
        dx, dg, db = capi.ln_bwd(dyd, xd, gd, mean32, rstd32, dtype)
    else:
        cf = bool(g["channel_first"])
        y, m, r = capi.in_fwd(xd, gd, bd, eps, dtype, cf)
        dx, dg, db = capi.in_bwd(dyd, xd, gd, mean32, rstd32, dtype, cf)
    torch.cuda.synchronize()
    assert_close(util.to_host(m), g["mean"], tol["stat"], "mean")
    assert_close(util.to_host(r), g["inv_std"], tol["stat"], "inv_std")
    assert_close(util.to_host(y), g["y"], tol["y"], "y")
    scale = util.dx_scale(g["dy"], np.sqrt(np.mean(g["gamma"].astype(np.float64) ** 2)), g["inv_std"], dtype)
    assert_close(util.to_host(dx), g["dx"], tol["dx"], "dx", scale=scale)
    assert_close(util.to_host(dg), g["dgamma"], tol["dw"], "dgamma")
    assert_close(util.to_host(db), g["dbeta"], tol["dw"], "dbeta")
