"""Host model, in numpy float32, of how the streaming kernels accumulate their statistics,
run on the data that breaks sums around a sampled pivot: a channel (or a thread's share of a
row) whose sampled elements sit 100 or 1000 standard deviations away from the bulk, e.g. the
zero-padded border of an image whose interior has a large mean.

* `pivot_sums`: S1 = sum(x - K), S2 = sum((x - K)^2), var = S2 / D - (S1 / D)^2 with K taken
  from the data.  It loses a factor (1 + (K - mean)^2 / var) of precision, so with an outlier
  pivot it misses the float32 tolerance of 1e-5.  Kept here as the negative control: it shows
  that the inputs below do separate a conditioned algorithm from an unconditioned one.
* `batch_welford`: what cl_fwd_stats (streaming variant) and chunk_wf do: every thread takes
  batches of B register-resident values, exact two-pass per batch, Chan update of its running
  (mean, m2, n) (the reference's Welford push, norm_util.h:182-211, is the B = 1 case); the
  workgroup combines its threads around the slab mean, and the slabs combine the same way
  around the instance mean (Chan's merge of all parts at once).
  It must stay within 1e-5 whatever the outliers.

The GPU tests of the same inputs are in test_gpu_conditioning.py.
"""
import numpy as np
import pytest

F = np.float32
EPS = 1e-3


def _seq_sum(a, axis):
    """Sequential float32 summation along an axis (numpy's cumsum does not pair up)."""
    return np.cumsum(a.astype(F), axis=axis, dtype=F).take(-1, axis=axis)


def pivot_sums(x, K, threads):
    """x: (D,) float32, D a multiple of threads.  Thread t owns x[t::threads]."""
    D = x.size
    d = (x.reshape(D // threads, threads) - F(K)).astype(F)
    s1 = _seq_sum(_seq_sum(d, 0), 0)
    s2 = _seq_sum(_seq_sum(d * d, 0), 0)
    dm = s1 / F(D)
    mean = F(K) + dm
    var = max(s2 / F(D) - dm * dm, F(0))
    return float(mean), float(var)


def batch_welford(x, threads, batch, slab_len):
    """x: (D,) float32; slabs of slab_len elements, inside a slab thread t owns
    slab[t::threads] and takes it `batch` values at a time."""
    D = x.size
    slabs = []
    for beg in range(0, D, slab_len):
        slab = x[beg:beg + slab_len]
        per_thread = slab.size // threads
        v = slab.reshape(per_thread, threads)
        mean = np.zeros(threads, F)
        m2 = np.zeros(threads, F)
        n = F(0)
        for b0 in range(0, per_thread, batch):
            f = v[b0:b0 + batch]
            nb = F(f.shape[0])
            mb = (_seq_sum(f, 0) * (F(1) / nb)).astype(F)
            q = _seq_sum(((f - mb) * (f - mb)).astype(F), 0)
            n_new = F(n + nb)
            w = F(nb / n_new)
            d = (mb - mean).astype(F)
            m2 = (m2 + (q + (d * d) * F(n * w))).astype(F)
            mean = (mean + d * w).astype(F)
            n = n_new
        slab_mean = F(_seq_sum((mean * n).astype(F), 0) / F(slab.size))
        dd = (mean - slab_mean).astype(F)
        slab_m2 = _seq_sum((m2 + n * (dd * dd)).astype(F), 0)
        slabs.append((slab_mean, slab_m2, F(slab.size)))
    # the slabs combine in two sweeps: mean = sum n_s mean_s / D, m2 = sum m2_s + n_s (mean_s - mean)^2
    s1 = F(0)
    for m, _, n in slabs:
        s1 = F(s1 + m * n)
    mean = F(s1 / F(D))
    m2 = F(0)
    for m, q, n in slabs:
        d = F(m - mean)
        m2 = F(m2 + F(q + n * F(d * d)))
    return float(mean), float(m2 / F(D))


def _rel_err_inv_std(var, x):
    ref = 1.0 / np.sqrt(x.astype(np.float64).var() + EPS)
    return abs(1.0 / np.sqrt(var + EPS) - ref) / ref


def _border_outliers(D, kappa, seed):
    """A channel of an image: bulk ~ N(kappa, 1), first / middle / last pixel 0."""
    rng = np.random.Generator(np.random.PCG64(seed))
    x = (rng.standard_normal(D) + kappa).astype(F)
    x[0] = x[D // 2] = x[D - 1] = 0
    return x


@pytest.mark.parametrize("kappa", [100.0, 1000.0])
def test_channels_last_streaming_model(kappa):
    D = 1 << 17
    x = _border_outliers(D, kappa, 7)
    K = float(np.median([x[0], x[D // 2], x[D - 1]]))
    assert K == 0.0
    _, var_pivot = pivot_sums(x, K, 32)
    mean, var = batch_welford(x, threads=32, batch=8, slab_len=4096)
    assert _rel_err_inv_std(var_pivot, x) > 1e-5          # the negative control fails
    assert _rel_err_inv_std(var, x) < 1e-6
    assert abs(mean - x.astype(np.float64).mean()) < 1e-6 * kappa


@pytest.mark.parametrize("kappa", [100.0, 1000.0])
def test_row_chunk_model(kappa):
    """chunk_wf: 256 threads, vectors of 8, batches of 4 vectors.  Four threads start on an
    outlier, which is the pivot of a sums formulation that shifts by the thread's first
    element; their share of the row then carries the whole loss."""
    D = 256 * 8 * 4 * 16
    rng = np.random.Generator(np.random.PCG64(8))
    x = (rng.standard_normal(D) + kappa).astype(F)
    x[np.arange(4) * 8] = 0                         # element 0 of vector t is thread t's first
    v = x.reshape(-1, 256, 8)                       # [iteration, thread, lane]
    if kappa >= 1000.0:
        # negative control: per-thread pivot sums, the threads then combined exactly (so that
        # only the per-thread loss shows)
        per_thread = np.transpose(v, (1, 0, 2)).reshape(256, -1)
        mu = x.astype(np.float64).mean()
        m2_pivot = 0.0
        for t in range(256):
            xt = per_thread[t]
            d = (xt - xt[0]).astype(F)
            s1 = _seq_sum(d, 0)
            s2 = _seq_sum(d * d, 0)
            m2_t = max(float(F(s2 - s1 * F(s1 / F(xt.size)))), 0.0)
            mean_t = float(xt[0]) + float(s1) / xt.size
            m2_pivot += m2_t + xt.size * (mean_t - mu) ** 2
        assert _rel_err_inv_std(m2_pivot / D, x) > 1e-5
    # batch model: a thread's 32 values of an iteration form one batch
    xt = np.ascontiguousarray(np.transpose(v.reshape(-1, 4, 256, 8), (0, 1, 3, 2)).reshape(-1, 256))
    _, var = batch_welford(xt.reshape(-1), threads=256, batch=32, slab_len=D)
    assert _rel_err_inv_std(var, x) < 1e-6
