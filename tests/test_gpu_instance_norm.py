"""GPU parity of the InstanceNorm entry points (through the C ABI) against the CPU oracle.

Shapes: benchmark configurations 3 and 4 (the latter with the spatial extent cut so the
oracle finishes in seconds) and the shape lists of the reference's own test
(tests/fused_instance_norm_test.py:145-170): N=2, C=32, rank 4 / 5 with 2^3..2^6 per
spatial dim, both layouts, plus the non-typical spatial extents.
"""
import numpy as np
import pytest

from oracle import oracle as O
from tests import util
from tests.util import TOL, assert_close

pytestmark = pytest.mark.gpu

EPS = 1e-3


@pytest.fixture(scope="module")
def capi():
    return util.Capi()


def run_case(capi, coracle, N, C, S, dtype, channel_first, seed_index, stddev=1.0, in_place=False):
    import torch

    print(f"IN case N={N} C={C} spatial={S} dtype={dtype} channel_first={channel_first} "
          f"seed={1000 + seed_index} in_place={in_place}", flush=True)
    x, gamma, beta, dy = util.in_inputs(N, C, S, dtype, channel_first, seed_index, stddev)
    y_ref, mean_ref, rstd_ref = coracle.in_fwd(x, gamma, beta, EPS, dtype, channel_first)

    xd = util.to_device(x, dtype)
    gd = torch.from_numpy(gamma).cuda()
    bd = torch.from_numpy(beta).cuda()
    x_keep = xd.clone() if in_place else xd
    y, mean, rstd = capi.in_fwd(xd, gd, bd, EPS, dtype, channel_first, y=xd if in_place else None)
    torch.cuda.synchronize()
    tol = TOL[dtype]
    assert_close(util.to_host(mean), mean_ref, tol["stat"], "mean")
    assert_close(util.to_host(rstd), rstd_ref, tol["stat"], "inv_std")
    assert_close(util.to_host(y), y_ref, tol["y"], "y")

    mean32 = mean_ref.astype(np.float32)
    rstd32 = rstd_ref.astype(np.float32)
    dx_ref, dg_ref, db_ref = coracle.in_bwd(dy, x, gamma, mean32.astype(np.float64),
                                            rstd32.astype(np.float64), dtype, channel_first)
    dyd = util.to_device(dy, dtype)
    dx, dg, db = capi.in_bwd(dyd, x_keep, gd, torch.from_numpy(mean32).cuda(),
                             torch.from_numpy(rstd32).cuda(), dtype, channel_first, dx=dyd if in_place else None)
    torch.cuda.synchronize()
    assert_close(util.to_host(dx), dx_ref, tol["dx"], "dx",
                 scale=util.dx_scale(dy, np.sqrt(np.mean(gamma.astype(np.float64) ** 2)), rstd32, dtype))
    assert_close(util.to_host(dg), dg_ref, tol["dw"], "dgamma")
    assert_close(util.to_host(db), db_ref, tol["dw"], "dbeta")


@pytest.mark.parametrize("channel_first", [False, True])
@pytest.mark.parametrize("dtype", ["f16", "f32", "bf16"])
def test_config3_2d(capi, coracle, dtype, channel_first):
    run_case(capi, coracle, 8, 64, 128 * 128, dtype, channel_first, 3)


@pytest.mark.parametrize("channel_first", [False, True])
def test_config4_3d_reduced(capi, coracle, channel_first):
    # [2,128,128,128,32] with the depth cut to 16: still a multi-workgroup reduction per (n,c)
    run_case(capi, coracle, 2, 32, 16 * 128 * 128, "f16", channel_first, 4)


@pytest.mark.parametrize("channel_first", [False, True])
@pytest.mark.parametrize("dtype", ["f16", "f32"])
@pytest.mark.parametrize("rank,d_exp", [(4, 3), (4, 4), (4, 5), (4, 6), (5, 3), (5, 4), (5, 5), (5, 6)])
def test_reference_shapes(capi, coracle, rank, d_exp, dtype, channel_first):
    # fused_instance_norm_test.py:145-155; x ~ N(0, 10^2) as there
    spatial = (2 ** d_exp) ** (rank - 2)
    run_case(capi, coracle, 2, 32, spatial, dtype, channel_first, 20, stddev=10.0)


@pytest.mark.parametrize("channel_first", [False, True])
@pytest.mark.parametrize("spatial", [1 * 11, 3 * 4, 1 * 31, 1 * 4001, 61 * 82, 113 * 145, 198 * 331, 179 * 2929])
def test_non_typical_spatial(capi, coracle, spatial, channel_first):
    # fused_instance_norm_test.py:157-179 (N=1, C=32, fp32)
    run_case(capi, coracle, 1, 32, spatial, "f32", channel_first, 21, stddev=10.0)


@pytest.mark.parametrize("channel_first", [False, True])
@pytest.mark.parametrize("dtype", ["f16", "f32"])
@pytest.mark.parametrize("C", [1, 3, 5, 9, 12, 17, 24, 48, 100, 255, 256, 520, 2049])
def test_channel_counts(capi, coracle, C, dtype, channel_first):
    # channel counts that are not a multiple of the vector width or not a power of two
    run_case(capi, coracle, 3, C, 777, dtype, channel_first, 22)


@pytest.mark.parametrize("channel_first", [False, True])
@pytest.mark.parametrize("dtype", ["f16", "f32"])
def test_in_place(capi, coracle, dtype, channel_first):
    run_case(capi, coracle, 2, 32, 4096, dtype, channel_first, 23, in_place=True)
    run_case(capi, coracle, 1, 8, 300000, dtype, channel_first, 23, in_place=True)
    # channel counts whose last vector overlaps its neighbour: the neighbour in the same wave
    # (268 = 33.5 vectors on 64 lanes), in the previous wave (516 = 64.5 vectors on 128 lanes),
    # streamed and register-resident slabs, single pass
    run_case(capi, coracle, 3, 268, 500, dtype, channel_first, 23, in_place=True)
    run_case(capi, coracle, 2, 516, 300, dtype, channel_first, 23, in_place=True)
    run_case(capi, coracle, 4, 100, 4096, dtype, channel_first, 23, in_place=True)
    run_case(capi, coracle, 40, 100, 60, dtype, channel_first, 23, in_place=True)
    run_case(capi, coracle, 2, 516, 40000, dtype, channel_first, 23, in_place=True)


@pytest.mark.parametrize("channel_first", [False, True])
@pytest.mark.parametrize("dtype", ["f32", "f16"])
@pytest.mark.parametrize("N,C,S", [(2, 32, 4096), (3, 24, 1000), (1, 8, 300000), (2, 64, 100)])
def test_unaligned_pointers(capi, coracle, N, C, S, dtype, channel_first):
    """Every array starts one element past an aligned address."""
    import torch

    print(f"IN unaligned N={N} C={C} spatial={S} dtype={dtype} channel_first={channel_first}", flush=True)
    x, gamma, beta, dy = util.in_inputs(N, C, S, dtype, channel_first, 26)
    y_ref, mean_ref, rstd_ref = coracle.in_fwd(x, gamma, beta, EPS, dtype, channel_first)
    xd, dyd = util.misalign(util.to_device(x, dtype)), util.misalign(util.to_device(dy, dtype))
    gd, bd = util.misalign(torch.from_numpy(gamma).cuda()), util.misalign(torch.from_numpy(beta).cuda())
    y, mean, rstd = capi.in_fwd(xd, gd, bd, EPS, dtype, channel_first, y=util.misalign(torch.empty_like(xd)))
    torch.cuda.synchronize()
    tol = TOL[dtype]
    assert_close(util.to_host(mean), mean_ref, tol["stat"], "mean")
    assert_close(util.to_host(rstd), rstd_ref, tol["stat"], "inv_std")
    assert_close(util.to_host(y), y_ref, tol["y"], "y")
    dx_ref, dg_ref, db_ref = coracle.in_bwd(dy, x, gamma, util.to_host(mean), util.to_host(rstd), dtype, channel_first)
    dx, dg, db = capi.in_bwd(dyd, xd, gd, util.misalign(mean), util.misalign(rstd), dtype, channel_first)
    torch.cuda.synchronize()
    assert_close(util.to_host(dx), dx_ref, tol["dx"], "dx",
                 scale=util.dx_scale(dy, np.sqrt(np.mean(gamma.astype(np.float64) ** 2)), util.to_host(rstd), dtype))
    assert_close(util.to_host(dg), dg_ref, tol["dw"], "dgamma")
    assert_close(util.to_host(db), db_ref, tol["dw"], "dbeta")


@pytest.mark.parametrize("dtype", ["f32", "f16"])
@pytest.mark.parametrize("N,C,S", [(64, 64, 27), (128, 40, 8), (16, 300, 30), (70, 64, 12)])
def test_tiny_spatial_channel_first(capi, coracle, N, C, S, dtype):
    """N * C >= 4096 planes of a few elements each: one thread per (n, c) plane."""
    run_case(capi, coracle, N, C, S, dtype, True, 27)


def test_layout_equivalence(capi):
    """IN over NC... of the transposed tensor equals the transpose of IN over N...C."""
    import torch

    x, gamma, beta, dy = util.in_inputs(2, 16, 1000, "f32", False, 24)
    gd, bd = torch.from_numpy(gamma).cuda(), torch.from_numpy(beta).cuda()
    x_cl = torch.from_numpy(x).cuda()
    x_cf = x_cl.permute(0, 2, 1).contiguous()
    y_cl, m_cl, r_cl = capi.in_fwd(x_cl, gd, bd, EPS, "f32", False)
    y_cf, m_cf, r_cf = capi.in_fwd(x_cf, gd, bd, EPS, "f32", True)
    torch.cuda.synchronize()
    assert_close(util.to_host(y_cf.permute(0, 2, 1).contiguous()), util.to_host(y_cl), 1e-5, "y")
    assert_close(util.to_host(m_cf), util.to_host(m_cl), 1e-5, "mean")
    assert_close(util.to_host(r_cf), util.to_host(r_cl), 1e-5, "inv_std")


def test_empty(capi):
    import torch

    L = capi.L
    dg = torch.full((4,), 7.0, device="cuda")
    db = torch.full((4,), 7.0, device="cuda")
    for layout in (0, 1):
        assert L.atexn_instance_norm_fwd(0, layout, None, None, None, 0, 4, 9, 1e-3, None, None, None, None, 0, None) == 0
        dg.fill_(7.0)
        db.fill_(7.0)
        assert L.atexn_instance_norm_bwd(0, layout, None, None, None, None, None, 0, 4, 9, None,
                                         dg.data_ptr(), db.data_ptr(), None, 0, None) == 0
        torch.cuda.synchronize()
        assert float(dg.abs().sum()) == 0.0 and float(db.abs().sum()) == 0.0


def test_deterministic(capi):
    import torch

    for cf in (False, True):
        x, gamma, beta, dy = util.in_inputs(4, 64, 4096, "f16", cf, 25)
        xd, dyd = util.to_device(x, "f16"), util.to_device(dy, "f16")
        gd, bd = torch.from_numpy(gamma).cuda(), torch.from_numpy(beta).cuda()
        outs = []
        for _ in range(2):
            y, m, r = capi.in_fwd(xd, gd, bd, EPS, "f16", cf)
            dx, dg, db = capi.in_bwd(dyd, xd, gd, m, r, "f16", cf)
            torch.cuda.synchronize()
            outs.append([t.clone() for t in (y, m, r, dx, dg, db)])
        for a, b in zip(*outs):
            assert torch.equal(a, b)


@pytest.mark.parametrize("N,C,S", [
    (1, 32, 216),      # a single instance: its sums are dgamma / dbeta directly
    (2, 32, 216),
    (600, 8, 20),      # 1 pixel slot per thread
    (600, 16, 200),    # 2
    (300, 64, 100),    # 4
    (40, 64, 250),     # 8
    (40, 128, 250),    # 16 forward, two stages backward
    (3, 4096, 4),      # two channel tiles
    (5, 520, 31),      # channel vectors not a power of two
    (600, 12, 20),     # channel counts that are not a multiple of the vector width: the last
    (64, 100, 64),     #   vector of a pixel overlaps its neighbour
    (2, 20, 216),
    (300, 36, 50),
    (1, 9, 1000),
    (3, 2051, 7),      # ... with two channel tiles
    (2, 320, 216),     # few instances: channel tiles of 8 vectors so that an instance fits and
    (2, 320, 512),     #   the launch has more workgroups (forward only at 512 pixels)
    (2, 100, 300),     # ... ragged, the last vector inside the second tile
    (3, 68, 200),      # ... ragged, the last vector reaching back into the first tile
    (5, 332, 128),     # ... ragged, six tiles
    (1, 64, 512),      # one workgroup in all
])
@pytest.mark.parametrize("dtype", ["f16", "f32"])
def test_channels_last_single_pass_matches_two_stage(coracle, N, C, S, dtype):
    """Instances that fit one workgroup's registers take single-pass kernels; the two-stage
    kernels stay reachable through the benchmark build's tuning hook.  Both must meet the
    oracle."""
    import torch

    capi = util.Capi(bench=True)
    x, gamma, beta, dy = util.in_inputs(N, C, S, dtype, False, 77)
    y_ref, m_ref, r_ref = coracle.in_fwd(x, gamma, beta, EPS, dtype, False)
    dx_ref, dg_ref, db_ref = coracle.in_bwd(dy, x, gamma, m_ref.astype(np.float32), r_ref.astype(np.float32),
                                            dtype, False)
    xd, dyd = util.to_device(x, dtype), util.to_device(dy, dtype)
    gd, bd = torch.from_numpy(gamma).cuda(), torch.from_numpy(beta).cuda()
    md = torch.from_numpy(m_ref.astype(np.float32)).cuda()
    rd = torch.from_numpy(r_ref.astype(np.float32)).cuda()
    tol = TOL[dtype]
    try:
        for fused in (1, 0):
            print(f"IN channels-last N={N} C={C} spatial={S} {dtype} single_pass={fused}", flush=True)
            assert capi.L.atexn_set_tuning(b"cl_fused", fused) == 0
            y, m, r = capi.in_fwd(xd, gd, bd, EPS, dtype, False)
            dx, dg, db = capi.in_bwd(dyd, xd, gd, md, rd, dtype, False)
            torch.cuda.synchronize()
            assert_close(util.to_host(m), m_ref, tol["stat"], "mean")
            assert_close(util.to_host(r), r_ref, tol["stat"], "inv_std")
            assert_close(util.to_host(y), y_ref, tol["y"], "y")
            scale = util.dx_scale(dy, np.sqrt(np.mean(gamma.astype(np.float64) ** 2)), r_ref, dtype)
            assert_close(util.to_host(dx), dx_ref, tol["dx"], "dx", scale=scale)
            assert_close(util.to_host(dg), dg_ref, tol["dw"], "dgamma")
            assert_close(util.to_host(db), db_ref, tol["dw"], "dbeta")
    finally:
        capi.L.atexn_set_tuning(b"cl_fused", 1)


@pytest.mark.parametrize("dtype", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("N,C,S,in_place", [(2, 4, 65536, False), (1, 3, 110592, False), (3, 2, 50176, True),
                                            (2, 2, 33001, False), (1, 5, 69632, False), (1, 2, 69633, False),
                                            (2, 3, 34816, True), (1, 2, 55299, False), (40, 16, 36864, False)])
def test_channel_first_planes_staged_on_chip(coracle, N, C, S, dtype, in_place):
    """Planes beyond the register-resident limit that still fit one workgroup's registers plus
    LDS make a single pass (forward up to 27 vectors per thread of 512, backward, which stages x
    and dy, up to 17): the limits of both directions for 16-bit and float32 planes, one
    element past them (two-stage kernels again), ragged planes, in place, and more planes than
    workgroups.  (The planner stages rows only when there are enough of them to fill the chip, and
    prefers the kernels that spread a plane over the workgroups of an XCD to these unless the call
    is in place or being captured; the benchmark build's tuning hook lifts the first condition
    and switches the other kernels off here.)"""
    capi = util.Capi(bench=True)
    assert capi.L.atexn_set_tuning(b"staged_rows", 2) == 0
    assert capi.L.atexn_set_tuning(b"plane_single", 0) == 0
    try:
        run_case(capi, coracle, N, C, S, dtype, True, 37, in_place=in_place)
    finally:
        assert capi.L.atexn_set_tuning(b"staged_rows", 1) == 0
        assert capi.L.atexn_set_tuning(b"plane_single", 1) == 0


@pytest.mark.parametrize("dtype", ["f16", "f32"])
@pytest.mark.parametrize("N,C,S", [(2, 2048, 64), (1, 4096, 40), (3, 520, 300), (2, 96, 5000), (1, 1048584, 3),
                                   (2, 300000, 5)])
def test_channels_last_wide_channel_counts(capi, coracle, N, C, S, dtype):
    """Few workgroups and thousands of channels: the dgamma / dbeta fold of the second backward
    stage deals its outputs out in chunks of adjacent columns."""
    run_case(capi, coracle, N, C, S, dtype, False, 29)


@pytest.mark.parametrize("dtype", ["f16", "f32"])
@pytest.mark.parametrize("N,C,S", [(16, 256, 8192), (9, 512, 4096), (20, 1024, 3000), (8, 8, 40000), (30, 16, 20000),
                                   (12, 64, 16 * 1024 + 5), (8, 100, 16384), (64, 100, 4096), (16, 20, 9000),
                                   (7, 13, 33333), (2, 128, 8000), (2, 320, 512), (2, 512, 2000), (3, 24, 2000),
                                   (1, 8, 300000)])
def test_channels_last_slab_fold_paths(capi, coracle, N, C, S, dtype):
    """The second stage folds the slab partials of its instance with all of a lane's partials in
    registers (at most 16 per lane, or 32 when the slab itself is register-resident) or in
    batches (more): shapes with one lane per channel and 17 .. 64 slabs, with 32 lanes per
    channel, with a short last slab, small instances whose slab count the planner caps at what
    the registers take (two sweeps of a 512-channel tile among them), and one instance of 235
    slabs, whose partials a launch of its own folds in batches that end in a partial one.  The
    backward cases deal the dgamma / dbeta columns out in chunks of 1, 4, 16 and 64."""
    run_case(capi, coracle, N, C, S, dtype, False, 31)


def _bits(t):
    import torch

    return t.view(torch.uint8)


@pytest.mark.parametrize("dtype", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("N,C,S", [(8, 64, 16384), (8, 32, 4096), (16, 64, 4000), (8, 128, 8192), (8, 24, 5000),
                                   (32, 64, 4096), (8, 64, 2048), (8, 256, 4096),
                                   # the XCD-major grid: batches that are no multiples of 8, more
                                   # workgroups than the chip holds, a single instance, many instances
                                   (4, 64, 16384), (16, 64, 16384), (2, 128, 4096), (1, 64, 8192), (3, 24, 5000),
                                   (100, 64, 2048), (5, 256, 4096),
                                   # more than two instances of 64 slabs per XCD: the backward built
                                   # for four workgroups per CU
                                   (20, 64, 16384)])
def test_channels_last_single_launch(coracle, N, C, S, dtype):
    """Register-resident slabs whose instance fits one XCD: statistics and their use run as ONE
    launch per direction whose workgroups exchange tagged partials while they run (every
    workgroup on the chip at once and N a multiple of 8: the (N, slabs, tiles) grid, dgamma / dbeta
    folded over the instances in the kernel; otherwise the XCD-major grid and a col_reduce over the
    instances).  Checked against the oracle, and three ways against itself through the benchmark
    build of the library (which can switch the path off and set the poll limit):
      * with a poll limit of 0 every workgroup gives up waiting at once and recomputes the other
        slabs itself: the outputs must have the bits of the normal run (the fallback is the same
        arithmetic), which is also what makes the results independent of timing;
      * two runs in a row on the same workspace (stale tags of the first call in place) agree;
      * the two-stage kernels (path switched off) meet the same oracle."""
    import torch

    capi = util.Capi(bench=True)
    L = capi.L
    x, gamma, beta, dy = util.in_inputs(N, C, S, dtype, False, 91)
    y_ref, m_ref, r_ref = coracle.in_fwd(x, gamma, beta, EPS, dtype, False)
    dx_ref, dg_ref, db_ref = coracle.in_bwd(dy, x, gamma, m_ref.astype(np.float32), r_ref.astype(np.float32),
                                            dtype, False)
    xd, dyd = util.to_device(x, dtype), util.to_device(dy, dtype)
    gd, bd = torch.from_numpy(gamma).cuda(), torch.from_numpy(beta).cuda()
    md = torch.from_numpy(m_ref.astype(np.float32)).cuda()
    rd = torch.from_numpy(r_ref.astype(np.float32)).cuda()
    tol = TOL[dtype]
    buf = __import__("ctypes").create_string_buffer(256)
    L.atexn_bench_describe_bwd(1, O.DTYPE_CODE[dtype], 1, N, C, S, buf, 256)
    print(f"IN channels-last single launch N={N} C={C} spatial={S} {dtype}: {buf.value.decode()}", flush=True)
    if b"cl_bwd_single" not in buf.value:
        pytest.skip("this shape and dtype stay on the two-stage kernels")

    def run():
        y, m, r = capi.in_fwd(xd, gd, bd, EPS, dtype, False)
        dx, dg, db = capi.in_bwd(dyd, xd, gd, md, rd, dtype, False)
        torch.cuda.synchronize()
        return y, m, r, dx, dg, db

    def check(out, what):
        y, m, r, dx, dg, db = out
        assert_close(util.to_host(m), m_ref, tol["stat"], what + " mean")
        assert_close(util.to_host(r), r_ref, tol["stat"], what + " inv_std")
        assert_close(util.to_host(y), y_ref, tol["y"], what + " y")
        scale = util.dx_scale(dy, np.sqrt(np.mean(gamma.astype(np.float64) ** 2)), r_ref, dtype)
        assert_close(util.to_host(dx), dx_ref, tol["dx"], what + " dx", scale=scale)
        assert_close(util.to_host(dg), dg_ref, tol["dw"], what + " dgamma")
        assert_close(util.to_host(db), db_ref, tol["dw"], what + " dbeta")

    names = ("y", "mean", "inv_std", "dx", "dgamma", "dbeta")
    try:
        normal = run()
        check(normal, "single launch")
        again = run()
        for n_, a, b in zip(names, normal, again):
            assert torch.equal(_bits(a), _bits(b)), f"second run differs in {n_}"
        # the builds for more workgroups per CU against the plain ones: the same arithmetic
        assert L.atexn_set_tuning(b"cl_single_occ", 0) == 0
        for n_, a, b in zip(names, normal, run()):
            assert torch.equal(_bits(a), _bits(b)), f"the plain build differs in {n_}"
        assert L.atexn_set_tuning(b"cl_single_occ", 1) == 0
        assert L.atexn_set_tuning(b"cl_single_polls", 0) == 0
        alone = run()
        check(alone, "single launch, poll limit 0")
        for n_, a, b in zip(names, normal, alone):
            assert torch.equal(_bits(a), _bits(b)), f"poll limit 0 differs from the normal run in {n_}"
        for polls in (1, 3, 8):  # some workgroups give up, others find what they wait for
            assert L.atexn_set_tuning(b"cl_single_polls", polls) == 0
            for n_, a, b in zip(names, normal, run()):
                assert torch.equal(_bits(a), _bits(b)), f"poll limit {polls} differs from the normal run in {n_}"
        assert L.atexn_set_tuning(b"cl_single_polls", 300) == 0
        # as after a call whose waits ran out: the waits of the next calls are cut short
        assert L.atexn_bench_mark_exchange_trouble(1) == 0
        for n_, a, b in zip(names, normal, run()):
            assert torch.equal(_bits(a), _bits(b)), f"short waits differ from the normal run in {n_}"
        assert L.atexn_bench_mark_exchange_trouble(0) == 0
        assert L.atexn_set_tuning(b"cl_single", 0) == 0
        check(run(), "two stages")
    finally:
        L.atexn_set_tuning(b"cl_single_polls", 300)
        L.atexn_set_tuning(b"cl_single", 1)
        L.atexn_set_tuning(b"cl_single_occ", 1)
        L.atexn_bench_mark_exchange_trouble(0)


def test_channels_last_single_launch_in_place_takes_two_stages(capi, coracle):
    """y written over x (dx over dy) keeps a call off the single-launch kernels, whose fallback
    reads other workgroups' parts of x: results as good as out of place."""
    run_case(capi, coracle, 8, 64, 16384, "f16", False, 92, in_place=True)


@pytest.mark.parametrize("dtype", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("N,C,S", [(8, 64, 16384), (8, 32, 4096), (16, 64, 3000), (64, 8, 32768), (2, 16, 5001),
                                   (24, 40, 2048), (8, 512, 8192),
                                   # lane groups per plane, several planes per workgroup and step
                                   (32, 128, 784), (2, 320, 216), (8, 512, 100), (64, 64, 196), (4, 256, 1000),
                                   (16, 1024, 64), (3, 128, 49)])
def test_channel_first_backward_folds_the_batch_in_the_row_kernel(coracle, N, C, S, dtype):
    """Channel-first planes with a workgroup each (or a group of lanes each, a workgroup then taking
    several consecutive planes per step), the planes of a channel on one XCD, at most 64 instances:
    the backward's row kernel publishes its plane sums as tagged pairs and the last workgroups of
    the grid add them up over the batch into dgamma / dbeta, instead of a col_reduce launch
    ((8, 512, 8192) has more workgroups than the chip holds at once).  Checked
    against the oracle and, through the benchmark build, against itself with the poll limit
    forced to 0 (every folding workgroup recomputes the plane sums of its channel itself: same
    bits), twice on the same workspace, and with the fold switched off (col_reduce again)."""
    import ctypes

    import torch

    capi = util.Capi(bench=True)
    L = capi.L
    buf = ctypes.create_string_buffer(384)
    L.atexn_bench_describe_bwd(1, O.DTYPE_CODE[dtype], 0, N, C, S, buf, 384)
    print(f"IN channel-first N={N} C={C} spatial={S} {dtype}: {buf.value.decode()}", flush=True)
    if b"folded over the batch in the kernel" not in buf.value:
        pytest.skip("this shape and dtype keep the col_reduce launch")
    x, gamma, beta, dy = util.in_inputs(N, C, S, dtype, True, 93)
    y_ref, m_ref, r_ref = coracle.in_fwd(x, gamma, beta, EPS, dtype, True)
    dx_ref, dg_ref, db_ref = coracle.in_bwd(dy, x, gamma, m_ref.astype(np.float32), r_ref.astype(np.float32),
                                            dtype, True)
    xd, dyd = util.to_device(x, dtype), util.to_device(dy, dtype)
    gd = torch.from_numpy(gamma).cuda()
    md = torch.from_numpy(m_ref.astype(np.float32)).cuda()
    rd = torch.from_numpy(r_ref.astype(np.float32)).cuda()
    tol = TOL[dtype]

    def run():
        out = capi.in_bwd(dyd, xd, gd, md, rd, dtype, True)
        torch.cuda.synchronize()
        return out

    def check(out, what):
        dx, dg, db = out
        scale = util.dx_scale(dy, np.sqrt(np.mean(gamma.astype(np.float64) ** 2)), r_ref, dtype)
        assert_close(util.to_host(dx), dx_ref, tol["dx"], what + " dx", scale=scale)
        assert_close(util.to_host(dg), dg_ref, tol["dw"], what + " dgamma")
        assert_close(util.to_host(db), db_ref, tol["dw"], what + " dbeta")

    try:
        normal = run()
        check(normal, "fold in the kernel")
        again = run()
        for n_, a, b in zip(("dx", "dgamma", "dbeta"), normal, again):
            assert torch.equal(_bits(a), _bits(b)), f"second run differs in {n_}"
        assert L.atexn_set_tuning(b"affine_fold_polls", 0) == 0
        alone = run()
        for n_, a, b in zip(("dx", "dgamma", "dbeta"), normal, alone):
            assert torch.equal(_bits(a), _bits(b)), f"poll limit 0 differs from the normal run in {n_}"
        assert L.atexn_set_tuning(b"affine_fold_polls", 2000) == 0
        assert L.atexn_set_tuning(b"affine_fold", 0) == 0
        check(run(), "col_reduce")
    finally:
        L.atexn_set_tuning(b"affine_fold_polls", 2000)
        L.atexn_set_tuning(b"affine_fold", 1)


def test_channel_first_backward_fold_with_more_workgroups_than_fit():
    """[8, 256, 32^3] fp16 channel-first: 1024 workgroups of 512 threads with 8 vectors per thread
    do not fit the chip at once.  The workgroups that fold the batch are the last of the grid, so
    they wait only for workgroups already started.  Checked against the same call with the fold
    switched off (col_reduce): dx to the bit, dgamma / dbeta to the summation-order tolerance."""
    import torch

    capi = util.Capi(bench=True)
    L = capi.L
    N, C, S = 8, 256, 32768
    gen = torch.Generator(device="cuda").manual_seed(97)
    x = (torch.randn(N, C, S, device="cuda", generator=gen) * 1.5 + 0.25).half()
    dy = torch.randn(N, C, S, device="cuda", generator=gen).half()
    gamma = torch.randn(C, device="cuda", generator=gen) * 0.5 + 1.0
    beta = torch.zeros(C, device="cuda")
    _, mean, rstd = capi.in_fwd(x, gamma, beta, EPS, "f16", True)
    try:
        folded = capi.in_bwd(dy, x, gamma, mean, rstd, "f16", True)
        torch.cuda.synchronize()
        assert L.atexn_set_tuning(b"affine_fold", 0) == 0
        plain = capi.in_bwd(dy, x, gamma, mean, rstd, "f16", True)
        torch.cuda.synchronize()
    finally:
        L.atexn_set_tuning(b"affine_fold", 1)
    assert torch.equal(_bits(folded[0]), _bits(plain[0])), "dx differs"
    for name, a, b in (("dgamma", folded[1], plain[1]), ("dbeta", folded[2], plain[2])):
        err = (a.double() - b.double()).abs().max().item()
        bound = 1e-5 * b.double().abs().max().item() + 1e-3
        assert err <= bound, f"{name}: {err} > {bound}"


@pytest.mark.parametrize("dtype", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("N,C,S", [(2, 8, 40000), (1, 3, 100000), (2, 4, 262144), (3, 5, 65544), (1, 16, 2097152),
                                   (2, 9, 32776), (1, 1, 1048576)])
def test_channel_first_planes_across_workgroups(coracle, N, C, S, dtype):
    """Channel-first planes too long for one workgroup (and too few, or too long, for the kernels
    that stage a plane in LDS): the chunks of a plane go to consecutive workgroups of one XCD, which
    keep them in registers and exchange their statistics while they run, so x (and dy) is read
    once.  Checked against the oracle, and through the benchmark build against itself with the
    poll limit forced to 0 (every workgroup recomputes the statistics of its plane's other chunks
    itself: same bits), twice on the same workspace, and with the path switched off (the two-stage
    kernels).  (1, 3, ...) and (2, 9, ...) leave XCDs with fewer planes than others."""
    import ctypes

    import torch

    capi = util.Capi(bench=True)
    L = capi.L
    buf = ctypes.create_string_buffer(384)
    L.atexn_bench_describe_bwd(1, O.DTYPE_CODE[dtype], 0, N, C, S, buf, 384)
    print(f"IN channel-first N={N} C={C} spatial={S} {dtype}: {buf.value.decode()}", flush=True)
    if b"plane_bwd_single" not in buf.value:
        pytest.skip("this shape and dtype take other kernels")
    x, gamma, beta, dy = util.in_inputs(N, C, S, dtype, True, 95)
    y_ref, m_ref, r_ref = coracle.in_fwd(x, gamma, beta, EPS, dtype, True)
    dx_ref, dg_ref, db_ref = coracle.in_bwd(dy, x, gamma, m_ref.astype(np.float32), r_ref.astype(np.float32),
                                            dtype, True)
    xd, dyd = util.to_device(x, dtype), util.to_device(dy, dtype)
    gd, bd = torch.from_numpy(gamma).cuda(), torch.from_numpy(beta).cuda()
    md = torch.from_numpy(m_ref.astype(np.float32)).cuda()
    rd = torch.from_numpy(r_ref.astype(np.float32)).cuda()
    tol = TOL[dtype]

    def run():
        y, m, r = capi.in_fwd(xd, gd, bd, EPS, dtype, True)
        dx, dg, db = capi.in_bwd(dyd, xd, gd, md, rd, dtype, True)
        torch.cuda.synchronize()
        return y, m, r, dx, dg, db

    def check(out, what):
        y, m, r, dx, dg, db = out
        assert_close(util.to_host(m), m_ref, tol["stat"], what + " mean")
        assert_close(util.to_host(r), r_ref, tol["stat"], what + " inv_std")
        assert_close(util.to_host(y), y_ref, tol["y"], what + " y")
        scale = util.dx_scale(dy, np.sqrt(np.mean(gamma.astype(np.float64) ** 2)), r_ref, dtype)
        assert_close(util.to_host(dx), dx_ref, tol["dx"], what + " dx", scale=scale)
        assert_close(util.to_host(dg), dg_ref, tol["dw"], what + " dgamma")
        assert_close(util.to_host(db), db_ref, tol["dw"], what + " dbeta")

    names = ("y", "mean", "inv_std", "dx", "dgamma", "dbeta")
    try:
        normal = run()
        check(normal, "one launch")
        again = run()
        for n_, a, b in zip(names, normal, again):
            assert torch.equal(_bits(a), _bits(b)), f"second run differs in {n_}"
        # the backward's build for three workgroups per CU (planes of more than 32 chunks) against
        # the one for two: the same arithmetic
        assert L.atexn_set_tuning(b"plane_single_occ", 0) == 0
        for n_, a, b in zip(names, normal, run()):
            assert torch.equal(_bits(a), _bits(b)), f"the build for two workgroups per CU differs in {n_}"
        assert L.atexn_set_tuning(b"plane_single_occ", 1) == 0
        assert L.atexn_set_tuning(b"plane_single_polls", 0) == 0
        alone = run()
        for n_, a, b in zip(names, normal, alone):
            assert torch.equal(_bits(a), _bits(b)), f"poll limit 0 differs from the normal run in {n_}"
        for polls in (1, 3, 8):  # some workgroups give up, others find what they wait for
            assert L.atexn_set_tuning(b"plane_single_polls", polls) == 0
            for n_, a, b in zip(names, normal, run()):
                assert torch.equal(_bits(a), _bits(b)), f"poll limit {polls} differs from the normal run in {n_}"
        assert L.atexn_set_tuning(b"plane_single_polls", 500) == 0
        # as after a call whose waits ran out: the waits of the next calls are cut short
        assert L.atexn_bench_mark_exchange_trouble(1) == 0
        for n_, a, b in zip(names, normal, run()):
            assert torch.equal(_bits(a), _bits(b)), f"short waits differ from the normal run in {n_}"
        assert L.atexn_bench_mark_exchange_trouble(0) == 0
        assert L.atexn_set_tuning(b"plane_single", 0) == 0
        check(run(), "two stages")
    finally:
        L.atexn_set_tuning(b"plane_single_polls", 500)
        L.atexn_set_tuning(b"plane_single", 1)
        L.atexn_set_tuning(b"plane_single_occ", 1)
        L.atexn_bench_mark_exchange_trouble(0)


def test_channel_first_planes_across_workgroups_in_place(capi, coracle):
    """y written over x (dx over dy) keeps such a call on the two-stage kernels (the one-launch
    kernels' fallback reads other workgroups' chunks of x): results as good as out of place."""
    run_case(capi, coracle, 2, 4, 262144, "f16", True, 96, in_place=True)


_DIGEST_SCRIPT = r"""
import hashlib, sys
import torch
sys.path.insert(0, sys.argv[1])
from tests import util
capi = util.Capi(bench=sys.argv[2] == "bench")
if sys.argv[2] == "bench":
    for name in (b"cl_single", b"plane_single", b"affine_fold"):
        assert capi.L.atexn_set_tuning(name, 0) == 0
h = hashlib.sha256()
for N, C, S, cf in ((8, 64, 16384, False), (16, 32, 4096, False), (2, 4, 262144, True), (8, 64, 16384, True)):
    gen = torch.Generator(device="cuda").manual_seed(1234 + N + S)
    shape = (N, C, S) if cf else (N, S, C)
    x = (torch.randn(shape, device="cuda", generator=gen) + 0.5).half()
    dy = torch.randn(shape, device="cuda", generator=gen).half()
    gamma = torch.rand(C, device="cuda", generator=gen) + 0.5
    beta = torch.randn(C, device="cuda", generator=gen)
    y, m, r = capi.in_fwd(x, gamma, beta, 1e-3, "f16", cf)
    dx, dg, db = capi.in_bwd(dy, x, gamma, m, r, "f16", cf)
    torch.cuda.synchronize()
    for t in (y, m, r, dx, dg, db):
        h.update(t.contiguous().view(torch.uint8).cpu().numpy().tobytes())
print("DIGEST", h.hexdigest())
"""


def test_exchange_kernels_can_be_switched_off_for_a_process():
    """ATEXN_NO_EXCHANGE=1 in the environment keeps every call of a process on the kernels that
    need no workgroups resident together (for processes that keep other kernels on the GPU all
    the time).  A child process with the variable set, calling the product library, must produce
    the bits that the benchmark build produces with those kernels switched off by its tuning hook
    (a second child, so that both see the same seeded inputs from a fresh process)."""
    import os
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

    def digest(flavour, extra_env):
        env = dict(os.environ, **extra_env)
        out = subprocess.run([sys.executable, "-c", _DIGEST_SCRIPT, root, flavour], env=env, capture_output=True,
                             text=True, timeout=300)
        assert out.returncode == 0, out.stderr[-2000:]
        lines = [ln for ln in out.stdout.splitlines() if ln.startswith("DIGEST ")]
        assert len(lines) == 1, out.stdout[-2000:]
        return lines[0]

    print("child processes: product library with ATEXN_NO_EXCHANGE=1, benchmark build with the switches off", flush=True)
    off_by_env = digest("product", {"ATEXN_NO_EXCHANGE": "1"})
    off_by_hook = digest("bench", {"ATEXN_NO_EXCHANGE": "0"})
    assert off_by_env == off_by_hook
