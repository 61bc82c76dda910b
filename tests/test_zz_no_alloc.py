"""atexn_layer_norm_bwd_static: the LayerNorm backward without a workspace argument (scratch in
a static device array of the library, nothing allocated by the call), against
atexn_layer_norm_bwd on the same inputs.  Both run the same kernels with the same launch plan,
so the results must be bit-identical.  Two calls in a row share the scratch array, the second
on a smaller problem, so stale contents of the first would show.
"""
import ctypes

import numpy as np
import pytest

from tests import util

pytestmark = pytest.mark.gpu

EPS = 1e-3


def _bwd_static(capi, dy, x, gamma, mean, rstd, dtype):
    import torch

    from oracle import oracle as O

    N, D = x.shape
    dx = torch.empty_like(x)
    dg = torch.empty(D, dtype=torch.float32, device=x.device)
    db = torch.empty(D, dtype=torch.float32, device=x.device)
    st = capi.L.atexn_layer_norm_bwd_static(
        O.DTYPE_CODE[dtype], dy.data_ptr(), x.data_ptr(), gamma.data_ptr(), mean.data_ptr(),
        rstd.data_ptr(), N, D, dx.data_ptr(), dg.data_ptr(), db.data_ptr(),
        torch.cuda.current_stream(x.device).cuda_stream)
    capi.capi.check(st)
    return dx, dg, db


def _same_bits(a, b):
    import torch

    return torch.equal(a.view(torch.uint8), b.view(torch.uint8))


@pytest.mark.parametrize("dtype,shapes", [
    ("f16", [(8192, 1024), (300, 1000)]),       # the BERT-large token shape, then a ragged one
    ("f32", [(4096, 512), (7, 33)]),
    ("bf16", [(64, 12288 // 4), (5, 8)]),
])
def test_static_scratch_matches_workspace_entry(dtype, shapes):
    import torch

    capi = util.Capi()
    for i, (N, D) in enumerate(shapes):
        print(f"no-alloc LN bwd dtype={dtype} N={N} D={D} call={i}", flush=True)
        x, gamma, beta, dy = util.ln_inputs("row_mean", N, D, dtype, 40 + i)
        xd, dyd = util.to_device(x, dtype), util.to_device(dy, dtype)
        gd, bd = torch.from_numpy(gamma).cuda(), torch.from_numpy(beta).cuda()
        _, mean, rstd = capi.ln_fwd(xd, gd, bd, EPS, dtype)
        dx_ref, dg_ref, db_ref = capi.ln_bwd(dyd, xd, gd, mean, rstd, dtype)
        torch.cuda.synchronize()
        dx, dg, db = _bwd_static(capi, dyd, xd, gd, mean, rstd, dtype)
        torch.cuda.synchronize()
        assert _same_bits(dx, dx_ref), "dx differs"
        assert _same_bits(dg, dg_ref), "dgamma differs"
        assert _same_bits(db, db_ref), "dbeta differs"


def test_static_scratch_limit_and_empty():
    import torch

    from oracle import oracle as O

    capi = util.Capi()
    L = capi.L
    limit = 8 << 20
    # [2048, 12288] fp16 needs one partial dgamma / dbeta row of 2 * 12288 floats per workgroup:
    # far more than the static buffer
    need = L.atexn_layer_norm_bwd_workspace_bytes(O.DTYPE_CODE["f16"], 2048, 12288)
    assert need > limit
    x = torch.zeros((2048, 12288), dtype=torch.float16, device="cuda")
    stat = torch.zeros(2048, dtype=torch.float32, device="cuda")
    w = torch.zeros(12288, dtype=torch.float32, device="cuda")
    with pytest.raises(capi.capi.InvalidArgumentError, match="static buffer"):
        _bwd_static(capi, x, x, w, stat, stat, "f16")
    # empty input: dgamma / dbeta are zero-filled, as by atexn_layer_norm_bwd
    g = torch.ones(16, dtype=torch.float32, device="cuda")
    dg = torch.full((16,), 7.0, device="cuda")
    db = torch.full((16,), 7.0, device="cuda")
    st = L.atexn_layer_norm_bwd_static(0, None, None, g.data_ptr(), None, None, 0, 16, None,
                                       dg.data_ptr(), db.data_ptr(),
                                       torch.cuda.current_stream().cuda_stream)
    capi.capi.check(st)
    torch.cuda.synchronize()
    assert float(dg.abs().max()) == 0.0 and float(db.abs().max()) == 0.0


def test_static_scratch_allocates_nothing_and_replays_from_a_graph():
    """The use the entry point exists for: one eager warm-up call (which looks the scratch
    address up), then the call recorded into a HIP graph and replayed.  Device memory in use
    does not move across an eager call (outputs are allocated beforehand), and every replay has
    the bits of atexn_layer_norm_bwd, with eager work and synchronisations between replays."""
    import torch

    from oracle import oracle as O

    capi = util.Capi()
    dtype, N, D = "f16", 2048, 1024
    print(f"no-alloc LN bwd under graph capture dtype={dtype} N={N} D={D}", flush=True)
    x, gamma, beta, dy = util.ln_inputs("row_mean", N, D, dtype, 44)
    xd, dyd = util.to_device(x, dtype), util.to_device(dy, dtype)
    gd, bd = torch.from_numpy(gamma).cuda(), torch.from_numpy(beta).cuda()
    _, mean, rstd = capi.ln_fwd(xd, gd, bd, EPS, dtype)
    dx_ref, dg_ref, db_ref = capi.ln_bwd(dyd, xd, gd, mean, rstd, dtype)
    dx = torch.empty_like(xd)
    dg = torch.empty(D, dtype=torch.float32, device="cuda")
    db = torch.empty(D, dtype=torch.float32, device="cuda")

    def call(stream):
        st = capi.L.atexn_layer_norm_bwd_static(
            O.DTYPE_CODE[dtype], dyd.data_ptr(), xd.data_ptr(), gd.data_ptr(), mean.data_ptr(),
            rstd.data_ptr(), N, D, dx.data_ptr(), dg.data_ptr(), db.data_ptr(), stream)
        capi.capi.check(st)

    call(torch.cuda.current_stream().cuda_stream)  # warm-up: the one-time symbol lookup
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    call(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before, (free_before, free_after)
    assert _same_bits(dx, dx_ref) and _same_bits(dg, dg_ref) and _same_bits(db, db_ref)

    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call(side.cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    with torch.cuda.graph(graph, stream=side):
        call(side.cuda_stream)
    for replay in range(3):
        for t in (dx, dg, db):
            t.fill_(float("nan"))
        junk = torch.randn(1 << 20, device="cuda").sum()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        del junk
        assert _same_bits(dx, dx_ref), f"replay {replay}: dx differs"
        assert _same_bits(dg, dg_ref), f"replay {replay}: dgamma differs"
        assert _same_bits(db, db_ref), f"replay {replay}: dbeta differs"
