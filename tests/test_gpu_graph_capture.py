"""The entry points only enqueue kernels on the caller's stream (no allocation, no
synchronisation, no memset nodes), so a forward + backward pair can be captured into a HIP
graph and replayed.  Each replay is checked bit for bit against the eager result, with
eager work and synchronisations between the replays."""
import numpy as np
import pytest

from tests import util

pytestmark = pytest.mark.gpu

EPS = 1e-3


@pytest.mark.parametrize("case", ["ln_resident", "ln_tiles", "ln_small", "ln_accumulators_in_lds", "in_channels_last",
                                  "in_channel_first", "in_channel_first_staged"])
def test_graph_replay_matches_eager(case):
    import torch

    capi = util.Capi()
    dtype = "f16"
    if case.startswith("ln"):
        N, D = {"ln_resident": (512, 1024), "ln_tiles": (6, 70001), "ln_small": (5000, 10),
                "ln_accumulators_in_lds": (300, 18432)}[case]
        x, gamma, beta, dy = util.ln_inputs("plain", N, D, dtype, 30)
        fwd = lambda xd, gd, bd: capi.ln_fwd(xd, gd, bd, EPS, dtype)  # noqa: E731
        bwd = lambda dyd, xd, gd, m, r: capi.ln_bwd(dyd, xd, gd, m, r, dtype)  # noqa: E731
    else:
        cf = case != "in_channels_last"
        # (staged: 512 planes of 36864 elements, two per CU, beyond the registers)
        N, C, S = (8, 64, 36864) if case == "in_channel_first_staged" else (4, 32, 4096)
        x, gamma, beta, dy = util.in_inputs(N, C, S, dtype, cf, 31)
        fwd = lambda xd, gd, bd: capi.in_fwd(xd, gd, bd, EPS, dtype, cf)  # noqa: E731
        bwd = lambda dyd, xd, gd, m, r: capi.in_bwd(dyd, xd, gd, m, r, dtype, cf)  # noqa: E731
    print(f"graph capture case={case}", flush=True)
    xd, dyd = util.to_device(x, dtype), util.to_device(dy, dtype)
    gd, bd = torch.from_numpy(gamma).cuda(), torch.from_numpy(beta).cuda()

    # eager reference
    y, m, r = fwd(xd, gd, bd)
    dx, dg, db = bwd(dyd, xd, gd, m, r)
    torch.cuda.synchronize()
    eager = [t.clone() for t in (y, m, r, dx, dg, db)]

    # capture on a side stream (torch's graph allocator serves the wrappers' torch.empty calls)
    graph = torch.cuda.CUDAGraph()
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        y, m, r = fwd(xd, gd, bd)  # warm-up on the capture stream
        bwd(dyd, xd, gd, m, r)
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    with torch.cuda.graph(graph):
        y, m, r = fwd(xd, gd, bd)
        dx, dg, db = bwd(dyd, xd, gd, m, r)
    outs = (y, m, r, dx, dg, db)
    for replay in range(3):
        for t in outs:
            t.fill_(float("nan")) if t.is_floating_point() else None
        # unrelated eager work and a synchronisation between the replays
        junk = torch.randn(1 << 20, device="cuda").sum()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        del junk
        for name, got, ref in zip(("y", "mean", "inv_std", "dx", "dgamma", "dbeta"), outs, eager):
            assert torch.equal(got, ref), f"replay {replay}: {name} differs from the eager result"
