"""Tensors with more than 2^31 elements (and one row longer than 2^31) through every kernel
family: the 288 GB of an MI355X hold them, so every element offset in the kernels must be
64-bit.  The CPU oracle would need minutes at these sizes, so the check is an independent
float64 evaluation of the closed forms with torch on the GPU, in chunks, over EVERY element
(the same closed forms the oracle is pinned against in test_oracle_pins.py), to the same
tolerances as the other fp16 tests."""
import pytest

from tests import util

pytestmark = pytest.mark.gpu

EPS = 1e-3
CHUNK = 1 << 26  # elements of a float64 working chunk


def _fill_normal(t, seed):
    import torch

    g = torch.Generator(device=t.device)
    g.manual_seed(seed)
    flat = t.view(-1)
    step = 1 << 30
    for i in range(0, flat.numel(), step):
        flat[i:i + step].normal_(generator=g)
    return t


def _close(got, ref, rtol, rms, what):
    import torch

    err = (got.double() - ref).abs()
    bound = rtol * ref.abs() + rtol * rms
    bad = err > bound
    if bool(bad.any()):
        idx = int(torch.nonzero(bad.view(-1))[0])
        raise AssertionError(f"{what}: first mismatch at flat index {idx} of the chunk: "
                             f"got {float(got.view(-1)[idx])} ref {float(ref.view(-1)[idx])}")


def _check_rows(x, dy, y, dx, mean, rstd, dg, db, gamma, beta, row_affine_C=0):
    """x, dy, y, dx: [R, D] fp16 on the GPU.  gamma / beta per column (LayerNorm) or, with
    row_affine_C = C, per row (channel-first InstanceNorm: row = n * C + c)."""
    import torch

    R, D = x.shape
    if row_affine_C:
        C = row_affine_C
        dg_ref = torch.zeros(C, dtype=torch.float64, device=x.device)
        db_ref = torch.zeros(C, dtype=torch.float64, device=x.device)
    else:
        dg_ref = torch.zeros(D, dtype=torch.float64, device=x.device)
        db_ref = torch.zeros(D, dtype=torch.float64, device=x.device)
    if D <= CHUNK // 4:
        rows = max(1, CHUNK // D)
        if row_affine_C:
            rows = max(row_affine_C, rows // row_affine_C * row_affine_C)
        for r0 in range(0, R, rows):
            r1 = min(R, r0 + rows)
            xf = x[r0:r1].double()
            m = xf.mean(1, keepdim=True)
            xc = xf - m
            r = torch.rsqrt((xc * xc).mean(1, keepdim=True) + EPS)
            xh = xc * r
            if row_affine_C:
                c = torch.arange(r0, r1, device=x.device) % row_affine_C
                gm, bt = gamma.double()[c][:, None], beta.double()[c][:, None]
            else:
                gm, bt = gamma.double()[None, :], beta.double()[None, :]
            _close(mean[r0:r1], m[:, 0], 1e-3, 1.0, f"mean rows {r0}..{r1}")
            _close(rstd[r0:r1], r[:, 0], 1e-3, 1.0, f"inv_std rows {r0}..{r1}")
            _close(y[r0:r1], xh * gm + bt, 1e-2, 1.0, f"y rows {r0}..{r1}")
            d = dy[r0:r1].double()
            g = d * gm
            s1 = g.sum(1, keepdim=True)
            s2 = (g * xh).sum(1, keepdim=True)
            _close(dx[r0:r1], r * (g - (s1 + xh * s2) / D), 1e-2, float(r.mean()), f"dx rows {r0}..{r1}")
            if row_affine_C:
                dg_ref += (d * xh).sum(1).view(-1, row_affine_C).sum(0)
                db_ref += d.sum(1).view(-1, row_affine_C).sum(0)
            else:
                dg_ref += (d * xh).sum(0)
                db_ref += d.sum(0)
    else:
        # few, very long rows: chunk along the columns, one pass per quantity
        cols = max(1, CHUNK // R)
        rng = [(c0, min(D, c0 + cols)) for c0 in range(0, D, cols)]

        def param(p, c0, c1):
            if row_affine_C:
                c = torch.arange(R, device=x.device) % row_affine_C
                return p.double()[c][:, None]
            return p[c0:c1].double()[None, :]

        s = torch.zeros(R, 1, dtype=torch.float64, device=x.device)
        for c0, c1 in rng:
            s += x[:, c0:c1].double().sum(1, keepdim=True)
        m = s / D
        s = torch.zeros_like(m)
        for c0, c1 in rng:
            xc = x[:, c0:c1].double() - m
            s += (xc * xc).sum(1, keepdim=True)
        r = torch.rsqrt(s / D + EPS)
        _close(mean, m[:, 0], 1e-3, 1.0, "mean")
        _close(rstd, r[:, 0], 1e-3, 1.0, "inv_std")
        s1 = torch.zeros_like(m)
        s2 = torch.zeros_like(m)
        for c0, c1 in rng:
            xh = (x[:, c0:c1].double() - m) * r
            g = dy[:, c0:c1].double() * param(gamma, c0, c1)
            s1 += g.sum(1, keepdim=True)
            s2 += (g * xh).sum(1, keepdim=True)
        for c0, c1 in rng:
            xh = (x[:, c0:c1].double() - m) * r
            gm, bt = param(gamma, c0, c1), param(beta, c0, c1)
            d = dy[:, c0:c1].double()
            _close(y[:, c0:c1], xh * gm + bt, 1e-2, 1.0, f"y cols {c0}..{c1}")
            _close(dx[:, c0:c1], r * (d * gm - (s1 + xh * s2) / D), 1e-2, float(r.mean()), f"dx cols {c0}..{c1}")
            if row_affine_C:
                dg_ref += (d * xh).sum(1).view(-1, row_affine_C).sum(0)
                db_ref += d.sum(1).view(-1, row_affine_C).sum(0)
            else:
                dg_ref[c0:c1] = (d * xh).sum(0)
                db_ref[c0:c1] = d.sum(0)
    rms = float(dg_ref.square().mean().sqrt())
    _close(dg, dg_ref, 1e-3, rms, "dgamma")
    _close(db, db_ref, 1e-3, float(db_ref.square().mean().sqrt()), "dbeta")


def _params(P, device):
    import torch

    g = torch.Generator(device=device)
    g.manual_seed(7)
    gamma = torch.empty(P, dtype=torch.float32, device=device).uniform_(0.5, 1.5, generator=g)
    beta = torch.empty(P, dtype=torch.float32, device=device).normal_(0.0, 0.1, generator=g)
    return gamma, beta


@pytest.mark.parametrize("N,D,family", [
    ((1 << 21) + 3, 1024, "one wave per row"),
    ((1 << 28) + 5, 10, "one thread per row"),
    ((1 << 18) + 1, 8200, "one workgroup per row, ragged"),
    (2, (1 << 31) + 9, "2-D tiles, a row longer than 2^31"),
    ((1 << 17) + 7, 16390, "backward with its accumulators in LDS, ragged"),
])
def test_layer_norm_beyond_int32(N, D, family):
    import torch

    capi = util.Capi()
    dev = "cuda:0"
    assert N * D > (1 << 31)
    print(f"LN beyond int32: N={N} D={D} ({family})", flush=True)
    x = _fill_normal(torch.empty((N, D), dtype=torch.float16, device=dev), 11)
    x[:, : min(D, 64)] += 1.5  # a non-zero row mean
    dy = _fill_normal(torch.empty((N, D), dtype=torch.float16, device=dev), 12)
    gamma, beta = _params(D, dev)
    y, mean, rstd = capi.ln_fwd(x, gamma, beta, EPS, "f16")
    dx, dg, db = capi.ln_bwd(dy, x, gamma, mean, rstd, "f16")
    torch.cuda.synchronize()
    _check_rows(x, dy, y, dx, mean, rstd, dg, db, gamma, beta)
    del x, dy, y, dx
    torch.cuda.empty_cache()


@pytest.mark.parametrize("N,C,D,family", [
    (512, 512, 8200, "planes in registers"),
    (2, 4, (1 << 28) + 3, "planes split over workgroups"),
    (64, 1024, 32780, "planes staged in registers and LDS"),
])
def test_instance_norm_channel_first_beyond_int32(N, C, D, family):
    import torch

    capi = util.Capi()
    dev = "cuda:0"
    assert N * C * D > (1 << 31)
    print(f"IN channel-first beyond int32: N={N} C={C} D={D} ({family})", flush=True)
    x = _fill_normal(torch.empty((N, C, D), dtype=torch.float16, device=dev), 21)
    dy = _fill_normal(torch.empty((N, C, D), dtype=torch.float16, device=dev), 22)
    gamma, beta = _params(C, dev)
    y, mean, rstd = capi.in_fwd(x, gamma, beta, EPS, "f16", True)
    dx, dg, db = capi.in_bwd(dy, x, gamma, mean, rstd, "f16", True)
    torch.cuda.synchronize()
    _check_rows(x.view(N * C, D), dy.view(N * C, D), y.view(N * C, D), dx.view(N * C, D),
                mean.view(-1), rstd.view(-1), dg, db, gamma, beta, row_affine_C=C)
    del x, dy, y, dx
    torch.cuda.empty_cache()


@pytest.mark.parametrize("N,D,C", [(3, (1 << 24) + 1, 64), (40000, 900, 60)])
def test_instance_norm_channels_last_beyond_int32(N, D, C):
    import torch

    capi = util.Capi()
    dev = "cuda:0"
    assert N * D * C > (1 << 31)
    print(f"IN channels-last beyond int32: N={N} D={D} C={C}", flush=True)
    x = _fill_normal(torch.empty((N, D, C), dtype=torch.float16, device=dev), 31)
    dy = _fill_normal(torch.empty((N, D, C), dtype=torch.float16, device=dev), 32)
    gamma, beta = _params(C, dev)
    y, mean, rstd = capi.in_fwd(x, gamma, beta, EPS, "f16", False)
    dx, dg, db = capi.in_bwd(dy, x, gamma, mean, rstd, "f16", False)
    torch.cuda.synchronize()
    gm, bt = gamma.double(), beta.double()
    dg_ref = torch.zeros(C, dtype=torch.float64, device=dev)
    db_ref = torch.zeros(C, dtype=torch.float64, device=dev)
    if D * C <= CHUNK:
        per = max(1, CHUNK // (D * C))
        for n0 in range(0, N, per):
            n1 = min(N, n0 + per)
            xf = x[n0:n1].double()
            m = xf.mean(1, keepdim=True)
            xc = xf - m
            r = torch.rsqrt((xc * xc).mean(1, keepdim=True) + EPS)
            xh = xc * r
            _close(mean[n0:n1], m[:, 0], 1e-3, 1.0, f"mean n {n0}..{n1}")
            _close(rstd[n0:n1], r[:, 0], 1e-3, 1.0, f"inv_std n {n0}..{n1}")
            _close(y[n0:n1], xh * gm + bt, 1e-2, 1.0, f"y n {n0}..{n1}")
            d = dy[n0:n1].double()
            g = d * gm
            s1 = g.sum(1, keepdim=True)
            s2 = (g * xh).sum(1, keepdim=True)
            _close(dx[n0:n1], r * (g - (s1 + xh * s2) / D), 1e-2, float(r.mean()), f"dx n {n0}..{n1}")
            dg_ref += (d * xh).sum((0, 1))
            db_ref += d.sum((0, 1))
    else:
        pix = max(1, CHUNK // C)
        rng = [(p0, min(D, p0 + pix)) for p0 in range(0, D, pix)]
        for n in range(N):
            s = torch.zeros(1, C, dtype=torch.float64, device=dev)
            for p0, p1 in rng:
                s += x[n, p0:p1].double().sum(0, keepdim=True)
            m = s / D
            s = torch.zeros_like(m)
            for p0, p1 in rng:
                xc = x[n, p0:p1].double() - m
                s += (xc * xc).sum(0, keepdim=True)
            r = torch.rsqrt(s / D + EPS)
            _close(mean[n], m[0], 1e-3, 1.0, f"mean n {n}")
            _close(rstd[n], r[0], 1e-3, 1.0, f"inv_std n {n}")
            s1 = torch.zeros_like(m)
            s2 = torch.zeros_like(m)
            for p0, p1 in rng:
                xh = (x[n, p0:p1].double() - m) * r
                g = dy[n, p0:p1].double() * gm
                s1 += g.sum(0, keepdim=True)
                s2 += (g * xh).sum(0, keepdim=True)
            for p0, p1 in rng:
                xh = (x[n, p0:p1].double() - m) * r
                d = dy[n, p0:p1].double()
                _close(y[n, p0:p1], xh * gm + bt, 1e-2, 1.0, f"y n {n} pixels {p0}..{p1}")
                _close(dx[n, p0:p1], r * (d * gm - (s1 + xh * s2) / D), 1e-2, float(r.mean()),
                       f"dx n {n} pixels {p0}..{p1}")
                dg_ref += (d * xh).sum(0)
                db_ref += d.sum(0)
    _close(dg, dg_ref, 1e-3, float(dg_ref.square().mean().sqrt()), "dgamma")
    _close(db, db_ref, 1e-3, float(db_ref.square().mean().sqrt()), "dbeta")
    del x, dy, y, dx
    torch.cuda.empty_cache()
