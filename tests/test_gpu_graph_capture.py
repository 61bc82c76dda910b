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

    # (two cases through the benchmark build with the kernels that would take their shapes in
    # eager mode, but not under capture, switched off: eager and replay then run the same ones;
    # test_graph_capture_of_a_single_launch_shape covers what happens otherwise)
    switch = {"in_channel_first_staged": b"plane_single", "in_channels_last": b"cl_single"}.get(case)
    capi = util.Capi(bench=switch is not None)
    if switch:
        assert capi.L.atexn_set_tuning(switch, 0) == 0
    try:
        _replay_matches_eager(capi, case)
    finally:
        if switch:
            assert capi.L.atexn_set_tuning(switch, 1) == 0


def _replay_matches_eager(capi, case):
    import torch

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


@pytest.mark.parametrize("N,C,S,cf", [(8, 64, 4096, False), (2, 4, 262144, True)])
def test_graph_capture_of_a_single_launch_shape(coracle, N, C, S, cf):
    """Shapes that run as one launch per direction in eager mode, with workgroups that exchange
    partials tagged with a per-call number (channels-last instances over the workgroups of an XCD;
    channel-first planes too long for one workgroup), are recorded as the two-stage kernels when
    the stream is being captured, since a replay would repeat the tag.  The replays must agree
    with each other bit for bit and with the oracle; against the eager (single-launch) result only
    the last bits of the statistics may differ (another order of the same additions)."""
    import torch

    from tests.util import TOL, assert_close

    capi = util.Capi()
    dtype = "f16"
    x, gamma, beta, dy = util.in_inputs(N, C, S, dtype, cf, 33)
    y_ref, m_ref, r_ref = coracle.in_fwd(x, gamma, beta, EPS, dtype, cf)
    print(f"graph capture of IN channel_first={cf} N={N} C={C} spatial={S} {dtype}", flush=True)
    xd, dyd = util.to_device(x, dtype), util.to_device(dy, dtype)
    gd, bd = torch.from_numpy(gamma).cuda(), torch.from_numpy(beta).cuda()
    y, m, r = capi.in_fwd(xd, gd, bd, EPS, dtype, cf)
    dx, dg, db = capi.in_bwd(dyd, xd, gd, m, r, dtype, cf)
    torch.cuda.synchronize()
    eager = [t.clone() for t in (y, m, r, dx, dg, db)]
    dx_ref, dg_ref, db_ref = coracle.in_bwd(dy, x, gamma, util.to_host(m), util.to_host(r), dtype, cf)

    graph = torch.cuda.CUDAGraph()
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        y, m, r = capi.in_fwd(xd, gd, bd, EPS, dtype, cf)
        capi.in_bwd(dyd, xd, gd, m, r, dtype, cf)
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    with torch.cuda.graph(graph):
        y, m, r = capi.in_fwd(xd, gd, bd, EPS, dtype, cf)
        dx, dg, db = capi.in_bwd(dyd, xd, gd, eager[1], eager[2], dtype, cf)
    outs = (y, m, r, dx, dg, db)
    first = None
    tol = TOL[dtype]
    for replay in range(3):
        for t in outs:
            t.fill_(float("nan"))
        junk = torch.randn(1 << 20, device="cuda").sum()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        del junk
        if first is None:
            first = [t.clone() for t in outs]
            assert_close(util.to_host(m), m_ref, tol["stat"], "mean")
            assert_close(util.to_host(r), r_ref, tol["stat"], "inv_std")
            assert_close(util.to_host(y), y_ref, tol["y"], "y")
            scale = util.dx_scale(dy, np.sqrt(np.mean(gamma.astype(np.float64) ** 2)), util.to_host(eager[2]), dtype)
            assert_close(util.to_host(dx), dx_ref, tol["dx"], "dx", scale=scale)
            assert_close(util.to_host(dg), dg_ref, tol["dw"], "dgamma")
            assert_close(util.to_host(db), db_ref, tol["dw"], "dbeta")
            assert_close(util.to_host(m), util.to_host(eager[1]), 1e-6, "mean vs eager")
            assert_close(util.to_host(r), util.to_host(eager[2]), 1e-6, "inv_std vs eager")
        else:
            for name, got, ref in zip(("y", "mean", "inv_std", "dx", "dgamma", "dbeta"), outs, first):
                assert torch.equal(got, ref), f"replay {replay}: {name} differs from the first replay"
