"""The kernels whose workgroups exchange results, beside a kernel that holds whole CUs.

A bounded busy kernel of the benchmark build (atexn_bench_occupy: 1024 threads and nearly all of
a CU's LDS per workgroup, gone after 20 ms at the latest) takes 192 of the 256 CUs on a second
stream; the InstanceNorm calls that run meanwhile find fewer places on an XCD than an instance has
slabs (a plane has chunks), so their waits run out for real: workgroups give up, claim and compute
what is missing, record the vain wait, and later waits are cut short.  Whatever the timing, the
outputs must have the bits of a run on the GPU alone."""
import os

import numpy as np
import pytest

from tests import util

pytestmark = pytest.mark.gpu

EPS = 1e-3
# random shapes beside the occupier; a longer sweep: ATEXN_SHARED_SEEDS=1000 python -m pytest tests/test_gpu_shared_gpu.py
N_SEEDS = int(os.environ.get("ATEXN_SHARED_SEEDS", "32"))


def _bits(t):
    import torch

    return t.view(torch.uint8)


@pytest.mark.parametrize("N,C,S,cf", [(8, 64, 16384, False), (16, 64, 16384, False), (2, 16, 2097152, True),
                                      (4, 32, 262144, True)])
def test_results_do_not_depend_on_who_else_runs(N, C, S, cf):
    import torch

    capi = util.Capi(bench=True)
    L = capi.L
    shape = (N, C, S) if cf else (N, S, C)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(77)
    x = torch.randn(shape, device="cuda", generator=gen).half()
    dy = torch.randn(shape, device="cuda", generator=gen).half()
    gamma = torch.rand(C, device="cuda", generator=gen) + 0.5
    beta = torch.randn(C, device="cuda", generator=gen) * 0.1
    side = torch.cuda.Stream()

    def run():
        y, m, r = capi.in_fwd(x, gamma, beta, EPS, "f16", cf)
        dx, dg, db = capi.in_bwd(dy, x, gamma, m, r, "f16", cf)
        return y, m, r, dx, dg, db

    alone = run()
    torch.cuda.synchronize()
    names = ("y", "mean", "inv_std", "dx", "dgamma", "dbeta")
    assert L.atexn_bench_mark_exchange_trouble(0) == 0
    recorded = 0
    try:
        for rep in range(4):
            torch.cuda.synchronize()
            assert L.atexn_bench_occupy(192, 20.0, side.cuda_stream) == 0
            torch.cuda._sleep(400000)  # the occupier gets its CUs first
            shared = run()
            torch.cuda.synchronize()
            for n_, a, b in zip(names, alone, shared):
                assert torch.equal(_bits(a), _bits(b)), f"run {rep} beside the occupier differs in {n_}"
            age = L.atexn_bench_exchange_trouble_age()
            recorded += 0 <= age < 64
    finally:
        torch.cuda.synchronize()
        L.atexn_bench_mark_exchange_trouble(0)
    # (how often a wait really ran out depends on where the occupier's workgroups landed: reported,
    # not required)
    print(f"IN N={N} C={C} spatial={S} {'channel-first' if cf else 'channels-last'}: "
          f"{recorded} of 4 runs beside the occupier recorded a wait that ran out", flush=True)


@pytest.mark.parametrize("seed", range(N_SEEDS))
def test_random_shapes_beside_the_occupier(seed):
    """Shapes of every kernel family that exchanges results (and a few that do not), in the three
    dtypes and both layouts: beside an occupier of 192 and of 128 CUs, the bits of a run alone."""
    import torch

    capi = util.Capi(bench=True)
    L = capi.L
    rng = np.random.Generator(np.random.PCG64(9000 + seed))
    cf = bool(rng.integers(0, 2))
    dtype = ["f16", "bf16", "f32"][int(rng.integers(0, 3))]
    if cf:
        N = int(rng.integers(1, 9))
        C = int(rng.choice([1, 3, 8, 16, 24, 32, 64]))
        S = int(rng.choice([40000, 65536, 100000, 131072, 262144, 524288, 1048576, 300008]))
        if N * C * S > 40_000_000:
            S = max(40000, 40_000_000 // (N * C) // 8 * 8)
    else:
        N = int(rng.integers(1, 40))
        C = int(rng.choice([8, 16, 24, 32, 48, 64, 96, 128, 256]))
        S = int(rng.choice([1024, 2000, 4096, 5000, 8192, 16384, 20000]))
        if N * C * S > 40_000_000:
            N = max(1, 40_000_000 // (C * S))
    shape = (N, C, S) if cf else (N, S, C)
    tdt = {"f16": torch.float16, "bf16": torch.bfloat16, "f32": torch.float32}[dtype]
    gen = torch.Generator(device="cuda")
    gen.manual_seed(1000 + seed)
    x = torch.randn(shape, device="cuda", generator=gen).to(tdt)
    dy = torch.randn(shape, device="cuda", generator=gen).to(tdt)
    gamma = torch.rand(C, device="cuda", generator=gen) + 0.5
    beta = torch.randn(C, device="cuda", generator=gen) * 0.1
    side = torch.cuda.Stream()
    print(f"IN {shape} {dtype} {'channel-first' if cf else 'channels-last'}", flush=True)

    def run():
        y, m, r = capi.in_fwd(x, gamma, beta, EPS, dtype, cf)
        dx, dg, db = capi.in_bwd(dy, x, gamma, m, r, dtype, cf)
        torch.cuda.synchronize()
        return y, m, r, dx, dg, db

    assert L.atexn_bench_mark_exchange_trouble(0) == 0
    alone = run()
    try:
        for wgs in (192, 128):
            for rep in range(2):
                torch.cuda.synchronize()
                assert L.atexn_bench_occupy(wgs, 6.0, side.cuda_stream) == 0
                torch.cuda._sleep(300000)
                shared = run()
                for n_, a, b in zip(("y", "mean", "inv_std", "dx", "dgamma", "dbeta"), alone, shared):
                    assert torch.equal(_bits(a), _bits(b)), f"beside {wgs} occupied CUs, run {rep}: {n_} differs"
    finally:
        torch.cuda.synchronize()
        L.atexn_bench_mark_exchange_trouble(0)


def test_the_occupier_leaves_in_time():
    import time

    import torch

    capi = util.Capi(bench=True)
    L = capi.L
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    assert L.atexn_bench_occupy(256, 5.0, torch.cuda.current_stream().cuda_stream) == 0
    torch.cuda.synchronize()
    took = time.perf_counter() - t0
    assert took < 0.5, f"a 5 ms occupier took {took * 1e3:.1f} ms"
    assert L.atexn_bench_occupy(0, 5.0, None) != 0 and L.atexn_bench_occupy(8, 1000.0, None) != 0
