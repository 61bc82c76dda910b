"""Re-entrancy: host threads calling the library at the same time on their own streams and
workspaces get the results a single thread gets, bit for bit (the library keeps no device
state; the reference's op is likewise called from concurrent executor threads on its stream,
fused_layer_norm_op.cu:830-835)."""
import threading

import numpy as np
import pytest

from tests import util

pytestmark = pytest.mark.gpu

EPS = 1e-3


def _work(capi, torch, kind, x, dy, gamma, beta, stream, out, key, reps):
    try:
        with torch.cuda.stream(stream):
            for _ in range(reps):
                if kind == "ln":
                    y, m, r = capi.ln_fwd(x, gamma, beta, EPS, "f16")
                    dx, dg, db = capi.ln_bwd(dy, x, gamma, m, r, "f16")
                else:
                    y, m, r = capi.in_fwd(x, gamma, beta, EPS, "f16", kind == "in_cf")
                    dx, dg, db = capi.in_bwd(dy, x, gamma, m, r, "f16", kind == "in_cf")
            stream.synchronize()
        out[key] = [t.clone() for t in (y, m, r, dx, dg, db)]
    except Exception as e:  # surfaced by the main thread
        out[key] = e


def test_concurrent_threads_and_streams():
    import torch

    capi = util.Capi()
    dev = "cuda:0"
    g = torch.Generator(device=dev)
    g.manual_seed(5)
    jobs = {
        "ln": ((4096, 1024), 1024),
        "ln_long": ((6, 70000), 70000),
        "in_cl": ((4, 64 * 64, 64), 64),
        "in_cf": ((4, 64, 64 * 64), 64),
        # batches of 8: the channels-last kernels whose workgroups exchange partial results while
        # they run (all of them must be on the chip, which two such launches at once contend for:
        # a wait that runs out makes a workgroup recompute its peers' share, to the same bits) and
        # the channel-first backward that folds its plane sums over the batch in the row kernel
        "in_cl_single": ((8, 128 * 128, 64), 64),
        "in_cf_fold": ((8, 64, 128 * 128), 64),
        # the same channels-last kernels on the XCD-major grid (a batch that is no multiple of 8)
        "in_cl_xm": ((5, 64 * 64, 64), 64),
        # channel-first planes spread over the workgroups of an XCD (16 chunks each)
        "in_cf_planes": ((2, 8, 64 * 64 * 128), 8),
    }
    data = {}
    for key, (shape, P) in jobs.items():
        x = torch.randn(shape, device=dev, dtype=torch.float32, generator=g).half()
        dy = torch.randn(shape, device=dev, dtype=torch.float32, generator=g).half()
        gamma = torch.rand(P, device=dev, generator=g) + 0.5
        beta = torch.randn(P, device=dev, generator=g) * 0.1
        data[key] = (x, dy, gamma, beta)
    torch.cuda.synchronize()

    def kind_of(key):
        return "ln" if key.startswith("ln") else key[:5]

    # single-threaded results on the default stream
    ref = {}
    for key, (x, dy, gamma, beta) in data.items():
        _work(capi, torch, kind_of(key), x, dy, gamma, beta, torch.cuda.current_stream(), ref, key, 1)
        assert not isinstance(ref[key], Exception), ref[key]

    print(f"concurrent threads: {len(data)} jobs x 2 threads each, own streams", flush=True)
    out = {}
    threads = []
    for key, (x, dy, gamma, beta) in data.items():
        for rep in range(2):
            s = torch.cuda.Stream(device=dev)
            s.wait_stream(torch.cuda.current_stream())
            t = threading.Thread(target=_work, args=(capi, torch, kind_of(key), x, dy, gamma, beta, s,
                                                     out, (key, rep), 40))
            threads.append(t)
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=120)
        assert not t.is_alive()
    torch.cuda.synchronize()
    for (key, rep), res in out.items():
        assert not isinstance(res, Exception), (key, rep, res)
        for got, want, name in zip(res, ref[key], ("y", "mean", "inv_std", "dx", "dgamma", "dbeta")):
            assert torch.equal(got, want), (key, rep, name)


def test_error_message_is_per_thread():
    """atexn_last_error is thread-local: a failure in one thread does not overwrite the
    message another thread reads."""
    capi = util.Capi()
    L = capi.L
    seen = {}

    def fail(tag, N):
        st = L.atexn_layer_norm_fwd(1, None, None, None, N, 8, 1e-3, None, None, None, None, 0, None)
        seen[tag] = (st, L.atexn_last_error().decode())

    t = threading.Thread(target=fail, args=("a", -5))
    t.start()
    t.join()
    st = L.atexn_layer_norm_fwd(99, None, None, None, 4, 8, 1e-3, None, None, None, None, 0, None)
    mine = L.atexn_last_error().decode()
    assert st == 1 and "dtype" in mine
    assert seen["a"][0] == 1 and "negative" in seen["a"][1]
