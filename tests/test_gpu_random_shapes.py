"""Seeded sweep over random shapes, dtypes, layouts, alignments and in-place use: every kernel
family and every boundary between them (resident / tiles / small / split / channels-last,
exact / non-exact / ragged) is crossed many times, each case checked against the oracle."""
import os

import numpy as np
import pytest

from tests import util
from tests.util import TOL, assert_close

pytestmark = pytest.mark.gpu

EPS = 1e-3
# cases per op; a longer sweep: ATEXN_RANDOM_SEEDS=1000 python -m pytest tests/test_gpu_random_shapes.py
N_SEEDS = int(os.environ.get("ATEXN_RANDOM_SEEDS", "48"))


def _pick_d(rng):
    kind = rng.integers(0, 6)
    if kind == 0:
        return int(rng.integers(1, 40))                       # tiny rows
    if kind == 1:
        return int(rng.integers(40, 1100))                    # sub-wave / one-wave rows
    if kind == 2:
        return int(8 * rng.integers(16, 2100))                # whole vectors, block-wide rows
    if kind == 3:
        return int(rng.integers(1100, 17000))                 # ragged block-wide rows
    if kind == 4:
        return int(rng.integers(16000, 40000))                # around the resident limits
    return int(rng.integers(40000, 300000))                   # long rows


def _check(got, ref, dy, gamma, rstd, dtype):
    y, m, r, dx, dg, db = got
    y_ref, m_ref, r_ref, dx_ref, dg_ref, db_ref = ref
    tol = TOL[dtype]
    assert_close(util.to_host(m), m_ref, tol["stat"], "mean")
    assert_close(util.to_host(r), r_ref, tol["stat"], "inv_std")
    assert_close(util.to_host(y), y_ref, tol["y"], "y")
    scale = util.dx_scale(dy, np.sqrt(np.mean(gamma.astype(np.float64) ** 2)), rstd, dtype)
    assert_close(util.to_host(dx), dx_ref, tol["dx"], "dx", scale=scale)
    assert_close(util.to_host(dg), dg_ref, tol["dw"], "dgamma")
    assert_close(util.to_host(db), db_ref, tol["dw"], "dbeta")


@pytest.mark.parametrize("seed", range(N_SEEDS))
def test_layer_norm_random(coracle, seed):
    import torch

    capi = util.Capi()
    rng = np.random.Generator(np.random.PCG64(5000 + seed))
    D = _pick_d(rng)
    budget = 3_000_000
    N = int(rng.integers(1, max(2, min(20000, budget // D))))
    if D <= 32 and rng.random() < 0.5:
        N = int(rng.integers(4096, 30000))                    # the thread-per-row kernels
    dtype = ["f32", "f16", "bf16"][int(rng.integers(0, 3))]
    mis = bool(rng.integers(0, 2))
    in_place = bool(rng.integers(0, 2))
    print(f"LN random seed={seed} N={N} D={D} dtype={dtype} misaligned={mis} in_place={in_place}", flush=True)
    x, gamma, beta, dy = util.ln_inputs("row_mean", N, D, dtype, 100 + seed)
    y_ref, m_ref, r_ref = coracle.ln_fwd(x, gamma, beta, EPS, dtype)
    wrap = util.misalign if mis else (lambda t: t)
    xd, dyd = wrap(util.to_device(x, dtype)), wrap(util.to_device(dy, dtype))
    gd, bd = wrap(torch.from_numpy(gamma).cuda()), wrap(torch.from_numpy(beta).cuda())
    x_keep = xd.clone() if in_place else xd
    y, m, r = capi.ln_fwd(xd, gd, bd, EPS, dtype, y=xd if in_place else None)
    torch.cuda.synchronize()
    dx_ref, dg_ref, db_ref = coracle.ln_bwd(dy, x, gamma, util.to_host(m), util.to_host(r), dtype)
    # dx may be written over dy (every other run)
    dx, dg, db = capi.ln_bwd(dyd, x_keep, gd, m, r, dtype, dx=dyd if seed % 2 else None)
    torch.cuda.synchronize()
    _check((y, m, r, dx, dg, db), (y_ref, m_ref, r_ref, dx_ref, dg_ref, db_ref), dy, gamma, util.to_host(r), dtype)


@pytest.mark.parametrize("seed", range(N_SEEDS))
def test_instance_norm_random(coracle, seed):
    import torch

    capi = util.Capi()
    rng = np.random.Generator(np.random.PCG64(7000 + seed))
    cf = bool(rng.integers(0, 2))
    C = int([rng.integers(1, 9), rng.integers(8, 70), 8 * rng.integers(1, 40), rng.integers(60, 600)][int(rng.integers(0, 4))])
    S = _pick_d(rng) if cf else int([rng.integers(1, 50), rng.integers(50, 5000), rng.integers(5000, 60000)][int(rng.integers(0, 3))])
    budget = 3_000_000
    N = int(rng.integers(1, max(2, min(64, budget // (C * S) + 1))))
    if C * S * N > 2 * budget:
        S = max(1, 2 * budget // (C * N))
    dtype = ["f32", "f16", "bf16"][int(rng.integers(0, 3))]
    mis = bool(rng.integers(0, 2))
    in_place = bool(rng.integers(0, 2))
    print(f"IN random seed={seed} N={N} C={C} spatial={S} dtype={dtype} channel_first={cf} misaligned={mis} "
          f"in_place={in_place}", flush=True)
    x, gamma, beta, dy = util.in_inputs(N, C, S, dtype, cf, 200 + seed)
    y_ref, m_ref, r_ref = coracle.in_fwd(x, gamma, beta, EPS, dtype, cf)
    wrap = util.misalign if mis else (lambda t: t)
    xd, dyd = wrap(util.to_device(x, dtype)), wrap(util.to_device(dy, dtype))
    gd, bd = wrap(torch.from_numpy(gamma).cuda()), wrap(torch.from_numpy(beta).cuda())
    x_keep = xd.clone() if in_place else xd
    y, m, r = capi.in_fwd(xd, gd, bd, EPS, dtype, cf, y=xd if in_place else None)
    torch.cuda.synchronize()
    dx_ref, dg_ref, db_ref = coracle.in_bwd(dy, x, gamma, util.to_host(m), util.to_host(r), dtype, cf)
    dx, dg, db = capi.in_bwd(dyd, x_keep, gd, m, r, dtype, cf, dx=dyd if seed % 2 else None)
    torch.cuda.synchronize()
    _check((y, m, r, dx, dg, db), (y_ref, m_ref, r_ref, dx_ref, dg_ref, db_ref), dy, gamma, util.to_host(r), dtype)


@pytest.mark.parametrize("seed", range(max(1, N_SEEDS // 2)))
def test_rows_kept_in_lds_random(coracle, seed):
    """The kernels that keep a row's accumulators, or part of the row itself, in LDS: LayerNorm
    rows of 8193 .. 21000 elements (the backward's accumulator kernel takes 16-bit rows from 16385
    and float32 rows from 8193 up to 20416 / 16384, the 2-D tiles beyond) and channel-first planes
    of 32769 .. 111000 elements with the staging forced on (few planes), at the edges of every
    range, ragged and misaligned.  Through the benchmark build of the library: only it can force
    the staging on."""
    import torch

    capi = util.Capi(bench=True)
    rng = np.random.Generator(np.random.PCG64(9000 + seed))
    dtype = ["f32", "f16", "bf16"][int(rng.integers(0, 3))]
    mis = bool(rng.integers(0, 2))
    in_place = bool(rng.integers(0, 2))
    wrap = util.misalign if mis else (lambda t: t)
    if seed % 2 == 0:
        D = int(rng.choice([rng.integers(8193, 21001), 8193, 16384, 16385, 20416, 20417, 18432, 12288]))
        N = int(rng.integers(1, 160))
        print(f"LN long-row random seed={seed} N={N} D={D} dtype={dtype} misaligned={mis} in_place={in_place}", flush=True)
        x, gamma, beta, dy = util.ln_inputs("row_mean", N, D, dtype, 300 + seed)
        y_ref, m_ref, r_ref = coracle.ln_fwd(x, gamma, beta, EPS, dtype)
        xd, dyd = wrap(util.to_device(x, dtype)), wrap(util.to_device(dy, dtype))
        gd, bd = wrap(torch.from_numpy(gamma).cuda()), wrap(torch.from_numpy(beta).cuda())
        x_keep = xd.clone() if in_place else xd
        y, m, r = capi.ln_fwd(xd, gd, bd, EPS, dtype, y=xd if in_place else None)
        torch.cuda.synchronize()
        dx_ref, dg_ref, db_ref = coracle.ln_bwd(dy, x, gamma, util.to_host(m), util.to_host(r), dtype)
        dx, dg, db = capi.ln_bwd(dyd, x_keep, gd, m, r, dtype, dx=dyd if in_place else None)
        torch.cuda.synchronize()
    else:
        S = int(rng.choice([rng.integers(32769, 111001), 32769, 69632, 69633, 110592, 34816, 34817, 55296, 55297]))
        # (at least four channels: a single dgamma that happens to cancel to almost nothing would
        # be held to a tolerance relative to itself)
        C = int(rng.integers(4, 9))
        N = int(rng.integers(1, 4))
        print(f"IN staged random seed={seed} N={N} C={C} spatial={S} dtype={dtype} misaligned={mis} in_place={in_place}", flush=True)
        x, gamma, beta, dy = util.in_inputs(N, C, S, dtype, True, 400 + seed)
        y_ref, m_ref, r_ref = coracle.in_fwd(x, gamma, beta, EPS, dtype, True)
        xd, dyd = wrap(util.to_device(x, dtype)), wrap(util.to_device(dy, dtype))
        gd, bd = wrap(torch.from_numpy(gamma).cuda()), wrap(torch.from_numpy(beta).cuda())
        x_keep = xd.clone() if in_place else xd
        assert capi.L.atexn_set_tuning(b"staged_rows", 2) == 0
        assert capi.L.atexn_set_tuning(b"plane_single", 0) == 0  # (they would take what is not in place)
        try:
            y, m, r = capi.in_fwd(xd, gd, bd, EPS, dtype, True, y=xd if in_place else None)
            torch.cuda.synchronize()
            dx_ref, dg_ref, db_ref = coracle.in_bwd(dy, x, gamma, util.to_host(m), util.to_host(r), dtype, True)
            dx, dg, db = capi.in_bwd(dyd, x_keep, gd, m, r, dtype, True, dx=dyd if in_place else None)
            torch.cuda.synchronize()
        finally:
            assert capi.L.atexn_set_tuning(b"staged_rows", 1) == 0
            assert capi.L.atexn_set_tuning(b"plane_single", 1) == 0
    _check((y, m, r, dx, dg, db), (y_ref, m_ref, r_ref, dx_ref, dg_ref, db_ref), dy, gamma, util.to_host(r), dtype)


@pytest.mark.parametrize("seed", range(max(1, N_SEEDS // 2)))
def test_exchange_paths_random(coracle, seed):
    """Shapes drawn for the kernels whose workgroups hand each other partial results while they
    run: channels-last instances whose slabs fit an XCD (one launch per direction, on either grid),
    channel-first planes with C a multiple of 8 (plane sums folded over the batch in the row
    kernel) and channel-first planes too long for a workgroup (a plane's chunks on consecutive
    workgroups of an XCD), at random sizes around their limits, misaligned tensors and in-place
    calls (which must take the other kernels) included.  Against the oracle."""
    import torch

    capi = util.Capi()
    rng = np.random.Generator(np.random.PCG64(11000 + seed))
    family = seed % 3
    cf = family != 0
    if family == 2:
        N = int(rng.integers(1, 4))
        C = int(rng.choice([1, 2, 3, 5, 8, 16]))
        S = int(rng.integers(32769, max(32770, 3_000_000 // (N * C))))
        if rng.integers(0, 4):
            S = S // 8 * 8  # whole vectors per plane: otherwise the two-stage kernels
        if rng.integers(0, 4) == 0:
            S = int(rng.integers(1, 9)) * 32768  # every workgroup's registers full
    else:
        # (batches that are multiples of 8 take the grid with an instance per XCD, the others the
        # XCD-major one)
        N = int(8 * rng.integers(1, 5)) if rng.integers(0, 2) else int(rng.integers(1, 65))
        C = int(8 * rng.integers(1, 17))
        budget = 4_000_000
        hi = max(600, budget // (N * C))
        S = int(rng.integers(max(300, hi // 8), hi))
        if cf and rng.integers(0, 2):
            S = S // 8 * 8  # whole vectors per plane
    dtype = ["f32", "f16", "bf16"][int(rng.integers(0, 3))]
    mis = bool(rng.integers(0, 3) == 0)
    in_place = bool(rng.integers(0, 4) == 0)
    print(f"IN exchange random seed={seed} N={N} C={C} spatial={S} dtype={dtype} channel_first={cf} "
          f"misaligned={mis} in_place={in_place}", flush=True)
    x, gamma, beta, dy = util.in_inputs(N, C, S, dtype, cf, 500 + seed)
    y_ref, m_ref, r_ref = coracle.in_fwd(x, gamma, beta, EPS, dtype, cf)
    wrap = util.misalign if mis else (lambda t: t)
    xd, dyd = wrap(util.to_device(x, dtype)), wrap(util.to_device(dy, dtype))
    gd, bd = wrap(torch.from_numpy(gamma).cuda()), wrap(torch.from_numpy(beta).cuda())
    x_keep = xd.clone() if in_place else xd
    y, m, r = capi.in_fwd(xd, gd, bd, EPS, dtype, cf, y=xd if in_place else None)
    torch.cuda.synchronize()
    dx_ref, dg_ref, db_ref = coracle.in_bwd(dy, x, gamma, util.to_host(m), util.to_host(r), dtype, cf)
    dx, dg, db = capi.in_bwd(dyd, x_keep, gd, m, r, dtype, cf, dx=dyd if in_place else None)
    torch.cuda.synchronize()
    _check((y, m, r, dx, dg, db), (y_ref, m_ref, r_ref, dx_ref, dg_ref, db_ref), dy, gamma, util.to_host(r), dtype)
