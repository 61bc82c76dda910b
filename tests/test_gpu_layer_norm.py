"""GPU parity of the LayerNorm entry points (through the C ABI) against the CPU oracle.

Shapes: the benchmark configurations at sizes the oracle finishes in seconds, plus the
shape lists of the reference's own test (tests/fused_layer_norm_test.py:118-151): powers
of two crossing every kernel family, odd sizes (element-wise paths and masked tails) and
the 'brittle' shapes with many rows.
"""
import numpy as np
import pytest

from tests import util
from tests.util import TOL, assert_close

pytestmark = pytest.mark.gpu

EPS = 1e-3


@pytest.fixture(scope="module")
def capi():
    return util.Capi()


def run_case(capi, coracle, cfg, N, D, dtype, seed_index, in_place=False):
    import torch

    print(f"LN case cfg={cfg} N={N} D={D} dtype={dtype} seed={1000 + seed_index} in_place={in_place}", flush=True)
    x, gamma, beta, dy = util.ln_inputs(cfg, N, D, dtype, seed_index)
    y_ref, mean_ref, rstd_ref = coracle.ln_fwd(x, gamma, beta, EPS, dtype, f64=True)

    xd = util.to_device(x, dtype)
    gd = torch.from_numpy(gamma).cuda()
    bd = torch.from_numpy(beta).cuda()
    x_keep = xd.clone() if in_place else xd
    y, mean, rstd = capi.ln_fwd(xd, gd, bd, EPS, dtype, y=xd if in_place else None)
    torch.cuda.synchronize()
    tol = TOL[dtype]
    assert_close(util.to_host(mean), mean_ref, tol["stat"], "mean")
    assert_close(util.to_host(rstd), rstd_ref, tol["stat"], "inv_std")
    assert_close(util.to_host(y), y_ref, tol["y"], "y")

    # backward takes the saved statistics as inputs: both sides get the same fp32 values
    mean32 = mean_ref.astype(np.float32)
    rstd32 = rstd_ref.astype(np.float32)
    dx_ref, dg_ref, db_ref = coracle.ln_bwd(dy, x, gamma, mean32.astype(np.float64),
                                            rstd32.astype(np.float64), dtype, f64=True)
    dyd = util.to_device(dy, dtype)
    dx, dg, db = capi.ln_bwd(dyd, x_keep, gd, torch.from_numpy(mean32).cuda(),
                             torch.from_numpy(rstd32).cuda(), dtype, dx=dyd if in_place else None)
    torch.cuda.synchronize()
    assert_close(util.to_host(dx), dx_ref, tol["dx"], "dx",
                 scale=util.dx_scale(dy, np.sqrt(np.mean(gamma.astype(np.float64) ** 2)), rstd32, dtype))
    # column sums of N terms: the absolute term scales with sqrt(N) like the sum itself
    assert_close(util.to_host(dg), dg_ref, tol["dw"], "dgamma")
    assert_close(util.to_host(db), db_ref, tol["dw"], "dbeta")


def test_config0_plumbing(capi, coracle):
    run_case(capi, coracle, "plain", 32, 1024, "f32", 0)


def test_config1_bert_large(capi, coracle):
    run_case(capi, coracle, "row_mean", 8192, 1024, "f16", 1)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("N,D", [(262144, 128), (16384, 4096), (2048, 12288)])
def test_config2_hidden_sweep(capi, coracle, N, D, dtype):
    # full widths at a reduced row count (a different launch plan: fewer rows per lane group,
    # smaller blocks); the full row counts run in test_gpu_full_size.py against the oracle
    n = min(N, 4096 if D <= 128 else 1024)
    run_case(capi, coracle, "scaled_rows", n, D, dtype, 2)


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("D", [16, 256, 1024, 2048, 4096, 8192, 16384, 32768, 65536, 2 ** 18])
@pytest.mark.parametrize("N", [1, 5])
def test_power_of_two_features(capi, coracle, N, D, dtype):
    run_case(capi, coracle, "plain", N, D, dtype, 10)


@pytest.mark.parametrize("dtype", ["f32", "f16"])
@pytest.mark.parametrize("D", [1, 3, 11, 12, 31, 100, 1000, 2003, 4001, 5002, 2 ** 14 + 1, 2 ** 16 + 2])
def test_non_typical_features(capi, coracle, D, dtype):
    run_case(capi, coracle, "plain", 2, D, dtype, 11)


@pytest.mark.parametrize("N,D", [(12000, 128 * 8 * 8), (1200, 128 * 8 * 6), (2, 128 * 8 * 8), (1, 64 * 384 * 276)])
def test_brittle_shapes(capi, coracle, N, D):
    # fused_layer_norm_test.py:144-151 ([12000,128,8,8] etc. with axis [1,2,3]); the first
    # is cut to 1500 rows to keep the oracle quick while still looping over many rows
    run_case(capi, coracle, "plain", min(N, 1500), D, "f32", 12)


@pytest.mark.parametrize("dtype", ["f32", "f16"])
@pytest.mark.parametrize("N,D", [(300, 1024), (7, 4096), (3, 40000), (2, 2 ** 18)])
def test_in_place(capi, coracle, N, D, dtype):
    # y may be forwarded onto x (fused_layer_norm_op.cc:337)
    run_case(capi, coracle, "plain", N, D, dtype, 13, in_place=True)


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("N,D", [(64, 1024), (37, 1000), (5, 8192), (3, 40000), (7, 40003), (2, 300001), (1000, 10),
                                 (500, 100), (300, 20000), (259, 24577), (11, 32761)])
def test_unaligned_pointers(capi, coracle, N, D, dtype):
    """Every array starts one element past an aligned address (a slice of a larger tensor):
    the 16-byte accesses of the kernels must not depend on pointer alignment."""
    import torch

    print(f"LN unaligned N={N} D={D} dtype={dtype}", flush=True)
    x, gamma, beta, dy = util.ln_inputs("plain", N, D, dtype, 16)
    y_ref, mean_ref, rstd_ref = coracle.ln_fwd(x, gamma, beta, EPS, dtype)
    xd, dyd = util.misalign(util.to_device(x, dtype)), util.misalign(util.to_device(dy, dtype))
    gd, bd = util.misalign(torch.from_numpy(gamma).cuda()), util.misalign(torch.from_numpy(beta).cuda())
    y, mean, rstd = capi.ln_fwd(xd, gd, bd, EPS, dtype, y=util.misalign(torch.empty_like(xd)))
    torch.cuda.synchronize()
    tol = TOL[dtype]
    assert_close(util.to_host(mean), mean_ref, tol["stat"], "mean")
    assert_close(util.to_host(rstd), rstd_ref, tol["stat"], "inv_std")
    assert_close(util.to_host(y), y_ref, tol["y"], "y")
    dx_ref, dg_ref, db_ref = coracle.ln_bwd(dy, x, gamma, util.to_host(mean), util.to_host(rstd), dtype)
    dx, dg, db = capi.ln_bwd(dyd, xd, gd, util.misalign(mean), util.misalign(rstd), dtype)
    torch.cuda.synchronize()
    assert_close(util.to_host(dx), dx_ref, tol["dx"], "dx",
                 scale=util.dx_scale(dy, np.sqrt(np.mean(gamma.astype(np.float64) ** 2)), util.to_host(rstd), dtype))
    assert_close(util.to_host(dg), dg_ref, tol["dw"], "dgamma")
    assert_close(util.to_host(db), db_ref, tol["dw"], "dbeta")


@pytest.mark.parametrize("dtype", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("N,D,in_place", [(600, 18432, False), (300, 20416, False), (1, 20000, False),
                                          (700, 16388, True), (257, 17001, False), (520, 12288, False),
                                          (9, 12291, True), (1500, 9000, False), (40, 16383, False)])
def test_backward_accumulators_in_lds(capi, coracle, N, D, dtype, in_place):
    """Rows of more than 2048 vectors whose dgamma / dbeta accumulators still fit a CU's LDS
    (up to 20416 elements: every 16-bit row from 16385 on, every float32 row from 8193 on)
    take a single-pass backward with the accumulators in LDS; ragged row ends (an overlapping
    last vector), a row count that is not a multiple of the workgroups, one row, the largest
    row, and dx written over dy."""
    run_case(capi, coracle, "plain", N, D, dtype, 19, in_place=in_place)


@pytest.mark.parametrize("dtype", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("N,D", [(300, 24576), (33, 24571), (700, 22528), (65, 12288), (64, 12285), (3, 24584)])
def test_forward_four_vectors_per_lane_wide(capi, coracle, N, D, dtype):
    """Rows of 2049 .. 3072 vectors run the forward with 4 vectors per lane on up to 768
    threads: the largest such row for either element size, ragged ends just below it, and the
    first row that goes back to 8 vectors per lane."""
    run_case(capi, coracle, "plain", N, D, dtype, 23)


@pytest.mark.parametrize("dtype", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("N,D", [(300, 16384), (65, 14336), (130, 13312), (64, 8192), (65, 7168), (3, 6656)])
def test_backward_four_vectors_per_lane(capi, coracle, N, D, dtype):
    """Rows of 1537 .. 2048 vectors run the backward with 4 vectors per lane and the next row
    prefetched (for float32 these are 6148 .. 8192 elements), exact multiples of the workgroup
    and not, more rows than workgroups and fewer."""
    run_case(capi, coracle, "plain", N, D, dtype, 29)


@pytest.mark.parametrize("dtype", ["f16", "f32"])
@pytest.mark.parametrize("N,D", [(10, 1000000), (100, 100000), (4, 400001), (3, 1000003), (1000, 40000),
                                 (300, 33000), (2, 2 ** 20 + 7)])
def test_long_rows(capi, coracle, N, D, dtype):
    """Rows beyond the register-resident limit, as in the reference's benchmark table
    (benchmarks/benchmark_layer_norm.py:53-63): few long rows, odd lengths included."""
    run_case(capi, coracle, "plain", N, D, dtype, 17)


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("N,D", [(5000, 4), (4096, 7), (5000, 8), (100000, 10), (4500, 13), (10000, 16), (4100, 31),
                                 (6000, 32), (7777, 25)])
def test_many_tiny_rows(capi, coracle, N, D, dtype):
    """Many rows of a few elements (one thread per row), as in the 10000000 x 10 line of the
    reference's benchmark table and the D = 11, 12, 16, 31 cases of its tests."""
    run_case(capi, coracle, "plain", N, D, dtype, 18)
    run_case(capi, coracle, "plain", N, D, dtype, 18, in_place=True)


def test_many_rows_narrow(capi, coracle):
    run_case(capi, coracle, "plain", 100000, 10, "f32", 14)
    run_case(capi, coracle, "plain", 50000, 100, "f16", 14)
    run_case(capi, coracle, "plain", 20000, 1000, "f16", 14)


def test_large_mean(capi, coracle):
    """x ~ U(10, 1000): the cancellation probe of fused_layer_norm_test.py:187-188."""
    import torch

    rng = util.rng_for(15)
    for dtype, N, D in (("f32", 64, 256), ("f32", 8, 5000), ("f32", 3, 100000)):
        x = rng.uniform(10.0, 1000.0, size=(N, D)).astype(np.float32)
        gamma, beta = util.affine_params(rng, D)
        y_ref, mean_ref, rstd_ref = coracle.ln_fwd(x, gamma, beta, EPS, dtype)
        y, mean, rstd = capi.ln_fwd(torch.from_numpy(x).cuda(), torch.from_numpy(gamma).cuda(),
                                    torch.from_numpy(beta).cuda(), EPS, dtype)
        torch.cuda.synchronize()
        assert_close(util.to_host(mean), mean_ref, 1e-5, "mean")
        assert_close(util.to_host(rstd), rstd_ref, 1e-5, "inv_std")
        assert_close(util.to_host(y), y_ref, 1e-5, "y")


def test_empty(capi):
    import torch

    L = capi.L
    dg = torch.full((8,), 7.0, device="cuda")
    db = torch.full((8,), 7.0, device="cuda")
    assert L.atexn_layer_norm_fwd(0, None, None, None, 0, 8, 1e-3, None, None, None, None, 0, None) == 0
    assert L.atexn_layer_norm_bwd(0, None, None, None, None, None, 0, 8, None, dg.data_ptr(),
                                  db.data_ptr(), None, 0, None) == 0
    torch.cuda.synchronize()
    assert float(dg.abs().sum()) == 0.0 and float(db.abs().sum()) == 0.0
    assert L.atexn_layer_norm_bwd(0, None, None, None, None, None, 0, 0, None, None, None, None, 0, None) == 0


def test_deterministic(capi):
    """Two runs give bit-identical results (no atomics anywhere on the path)."""
    import torch

    x, gamma, beta, dy = util.ln_inputs("row_mean", 4096, 1024, "f16", 16)
    xd, dyd = util.to_device(x, "f16"), util.to_device(dy, "f16")
    gd, bd = torch.from_numpy(gamma).cuda(), torch.from_numpy(beta).cuda()
    outs = []
    for _ in range(2):
        y, m, r = capi.ln_fwd(xd, gd, bd, EPS, "f16")
        dx, dg, db = capi.ln_bwd(dyd, xd, gd, m, r, "f16")
        torch.cuda.synchronize()
        outs.append([t.clone() for t in (y, m, r, dx, dg, db)])
    for a, b in zip(*outs):
        assert torch.equal(a, b)
