#!/usr/bin/env python3
"""Benchmark of the fused LayerNorm / InstanceNorm forward + backward on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--case NAME] [--no-cpu] [--cold-only]

One "step" is one forward plus one backward call of the hot path (kernel-level C ABI of
libatex_norms_hip.so) over one batch of synthetic input that is already resident in HBM.
The default case is the LayerNorm BERT-large token shape, x fp16 [8192, 1024].

Cache honesty: the 16.8 MB tensors of that case would sit in the 256 MB Infinity Cache if
every step reused them, so the timed loop rotates over enough independent buffer sets
(x, dy, y, dx, statistics) that a set's lines were last touched more than 512 MB ago.

Output: ONE JSON line on stdout.
  value        algorithmic bytes of fwd + bwd / wall time per step, in GB/s
  roofline     the dominant kernel (the backward row kernel), timed alone with events on the
               launch stream: algorithmic bytes of the backward / its average duration,
               against the 8 TB/s HBM peak.  "Alone" needs the benchmark build of the library
               (libatex_norms_hip_bench.so, same sources plus a switch that skips the column
               reduction); every other figure comes from the product library
  targets      (default case only) the second target shape, InstanceNorm x fp16 [8,128,128,64]
               in both layouts: us per call, GB/s, fraction of peak, roofline of its backward
  configs      (default case only) every other benchmark configuration -- the fp32 [32,1024]
               plumbing case, the hidden-size sweep in fp16 and bf16, the 3-D volume in both
               layouts -- each with us per call (fwd, bwd, fwd+bwd), GB/s, % of peak and torch's
               copy / add on the same tensors as streaming references
  cpu_baseline the C oracle's float flavour (OpenMP over rows) on the same workload, timed
               on this machine's host cores; `unfused_composite` inside it is the unfused op
               sequence a framework would run instead (torch on the CPU, autograd backward)
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
ROTATE_BYTES = 640 << 20  # footprint the buffer rotation must exceed

# name -> (op, dtype, dims); LayerNorm dims = (N, D); InstanceNorm dims = (N, C, D, channel_first)
CASES = {
    "ln_cfg0": ("ln", "f32", (32, 1024)),
    "ln_bert": ("ln", "f16", (8192, 1024)),
    "ln_128_f16": ("ln", "f16", (262144, 128)),
    "ln_128_bf16": ("ln", "bf16", (262144, 128)),
    "ln_4096_f16": ("ln", "f16", (16384, 4096)),
    "ln_4096_bf16": ("ln", "bf16", (16384, 4096)),
    "ln_12288_f16": ("ln", "f16", (2048, 12288)),
    "ln_12288_bf16": ("ln", "bf16", (2048, 12288)),
    "in2d_nhwc": ("in", "f16", (8, 64, 128 * 128, False)),
    "in2d_nchw": ("in", "f16", (8, 64, 128 * 128, True)),
    "in3d_ndhwc": ("in", "f16", (2, 32, 128 ** 3, False)),
    "in3d_ncdhw": ("in", "f16", (2, 32, 128 ** 3, True)),
    # shapes of the reference's own benchmark tables (benchmark_layer_norm.py:53-63,
    # benchmark_instance_norm.py:58-69), not part of --case all
    "ln_8192x1024_f32": ("ln", "f32", (8192, 1024)),
    "ln_8192x2048_f16": ("ln", "f16", (8192, 2048)),
    "ln_8192x768_f16": ("ln", "f16", (8192, 768)),
    "ln_8192x1536_f16": ("ln", "f16", (8192, 1536)),
    "in2d_nhwc_f32": ("in", "f32", (8, 64, 128 * 128, False)),
    "in2d_nchw_f32": ("in", "f32", (8, 64, 128 * 128, True)),
    "ln_8192x10240": ("ln", "f16", (8192, 10240)),
    "ln_4096x16384": ("ln", "f16", (4096, 16384)),
    "lnref_10x1e7": ("ln", "f16", (10, 10000000)),
    "lnref_100x1e6": ("ln", "f16", (100, 1000000)),
    "lnref_1e3x1e5": ("ln", "f16", (1000, 100000)),
    "lnref_1e4x1e4": ("ln", "f16", (10000, 10000)),
    "lnref_1e5x1e3": ("ln", "f16", (100000, 1000)),
    "lnref_1e6x100": ("ln", "f16", (1000000, 100)),
    "lnref_1e7x10": ("ln", "f16", (10000000, 10)),
    "lnref_4x400001": ("ln", "f16", (4, 400001)),
    "lnref_4x10000001": ("ln", "f16", (4, 10000001)),
    "in_1x128x512x512_cl": ("in", "f16", (1, 128, 512 * 512, False)),
    "in_1x32x128x128x128_cl": ("in", "f16", (1, 32, 128 ** 3, False)),
    "inref_8x64x64_cl": ("in", "f16", (8, 64, 64 ** 3, False)),
    "inref_8x64x64_cf": ("in", "f16", (8, 64, 64 ** 3, True)),
    "inref_8x128x64_cl": ("in", "f16", (8, 128, 64 ** 3, False)),
    "inref_8x128x64_cf": ("in", "f16", (8, 128, 64 ** 3, True)),
    "inref_4x256x32_cl": ("in", "f16", (4, 256, 32 ** 3, False)),
    "inref_4x256x32_cf": ("in", "f16", (4, 256, 32 ** 3, True)),
    # few instances, hundreds of channels (the deep levels of a 3-D U-Net), and few long rows
    "in_2x320x216_cl": ("in", "f16", (2, 320, 6 ** 3, False)),
    "in_2x320x512_cl": ("in", "f16", (2, 320, 8 ** 3, False)),
    "in_2x128x4096_cl": ("in", "f16", (2, 128, 16 ** 3, False)),
    "ln_512x4096_f16": ("ln", "f16", (512, 4096)),
    # rows of 3072 float32 vectors: the backward keeps its dgamma / dbeta accumulators in LDS
    "ln_8192x12288_f32": ("ln", "f32", (8192, 12288)),
    # 1024 channel-first planes of 256 x 256: staged in registers + LDS, single pass
    "in_16x64x256x256_cf": ("in", "f16", (16, 64, 256 * 256, True)),
    # more instances than the chip holds workgroups for at once: the channels-last single-launch
    # kernels on their XCD-major grid
    "in_16x128x128x64_cl": ("in", "f16", (16, 64, 128 * 128, False)),
    "in_64x128x128x64_cl": ("in", "f16", (64, 64, 128 * 128, False)),
    # the InstanceNorm configurations in bf16 (the configurations name fp16; the ops take both)
    "in2d_nhwc_bf16": ("in", "bf16", (8, 64, 128 * 128, False)),
    "in2d_nchw_bf16": ("in", "bf16", (8, 64, 128 * 128, True)),
    "in3d_ndhwc_bf16": ("in", "bf16", (2, 32, 128 ** 3, False)),
    "in3d_ncdhw_bf16": ("in", "bf16", (2, 32, 128 ** 3, True)),
}
# cases that `--case all` leaves out (single-purpose sweeps and the reference's benchmark table)
SWEEP_ONLY_CASES = frozenset(
    [n for n in CASES if n.startswith(("lnref_", "inref_", "in_1x", "in_16x", "in_64x", "ln_8192x", "ln_4096x")) or n.endswith("_f32") or (n.startswith("in") and n.endswith("_bf16"))])
DEFAULT_CASE = "ln_bert"
# the two shapes the throughput target is stated on, reported on the default run's line
TARGET_CASES = ("ln_bert", "in2d_nhwc", "in2d_nchw")

# Bytes between L2 and memory per launch of the kernel(s) the roofline object is quoted on,
# from `rocprofv3 --pmc FETCH_SIZE` and `--pmc WRITE_SIZE` runs of this file, each scaled by
# what the same counter reads for the 64 MiB negation of --copy-calibration (FETCH_SIZE x 2.0,
# WRITE_SIZE x 1.0).  Summaries: profiles/<case>_hbm_traffic.txt.  Cases without a run: None.
MEASURED_TRAFFIC = {
    "ln_bert": 52.79e6,                 # rows_bwd_resident
    "ln_128_f16": 203.73e6,             # rows_bwd_resident
    "ln_4096_f16": 412.22e6,            # rows_bwd_resident
    "ln_12288_f16": 176.84e6,           # rows_bwd_resident (151.0 MB of rows + 25.2 MB of partial rows)
    "in2d_nchw": 50.58e6,               # rows_bwd_resident (row-affine, plane sums folded in the kernel)
    "in2d_nhwc": 51.71e6,               # cl_bwd_single
    "in3d_ndhwc": 536.94e6 + 805.87e6,  # cl_bwd_sums + cl_bwd_apply
    "in3d_ncdhw": 813.19e6,             # plane_bwd_single (plane sums folded in the kernel)
}
ESIZE = {"f32": 4, "f16": 2, "bf16": 2}


def algorithmic_bytes(op, dtype, dims):
    """(fwd, bwd) bytes every implementation must move: x in, y out, the fp32 parameters and
    statistics; dy and x in, dx out, statistics in, dgamma / dbeta out."""
    s = ESIZE[dtype]
    if op == "ln":
        N, D = dims
        return 2 * N * D * s + 8 * D + 8 * N, 3 * N * D * s + 12 * D + 8 * N
    N, C, D, _ = dims
    return 2 * N * C * D * s + 8 * C + 8 * N * C, 3 * N * C * D * s + 12 * C + 8 * N * C


def _storage(a, dtype):
    from oracle import oracle as O

    return O.to_storage(a, dtype)


def make_host_inputs(op, dtype, dims, seed):
    rng = np.random.Generator(np.random.PCG64(seed))
    if op == "ln":
        N, D = dims
        x = rng.standard_normal((N, D), dtype=np.float32)
        x += rng.uniform(-2, 2, size=(N, 1)).astype(np.float32)
        dy = rng.standard_normal((N, D), dtype=np.float32)
        P = D
    else:
        N, C, D, cf = dims
        shape = (N, C, D) if cf else (N, D, C)
        x = rng.standard_normal(shape, dtype=np.float32)
        dy = rng.standard_normal(shape, dtype=np.float32)
        P = C
    gamma = rng.uniform(0.5, 1.5, size=P).astype(np.float32)
    beta = (rng.standard_normal(P) * 0.1).astype(np.float32)
    return x, gamma, beta, dy


# --tune given: every measurement goes through the benchmark build (the product library has no
# launch-planning switches)
USE_BENCH_LIB_EVERYWHERE = False


def bench_lib():
    """The benchmark build of the library (launch-planning switches, among them "bwd_stage_mask",
    and the plan description), or None when it has not been built."""
    from atex_amd.nv_norms import _capi

    try:
        return _capi.bench_lib()
    except ImportError:
        return None


class GpuCase:
    """Device buffers of one case, R rotating sets, and closures that launch fwd / bwd."""

    def __init__(self, op, dtype, dims, device="cuda:0"):
        import torch

        from atex_amd.nv_norms import _capi

        self.torch = torch
        self.capi = _capi
        self.L = bench_lib() if USE_BENCH_LIB_EVERYWHERE else _capi.lib()
        self.op, self.dtype, self.dims = op, dtype, dims
        self.code = {"f32": 0, "f16": 1, "bf16": 2}[dtype]
        tdt = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[dtype]
        if op == "ln":
            N, D = dims
            shape, stat_shape, P = (N, D), (N,), D
            self.fwd_ws = self.L.atexn_layer_norm_fwd_workspace_bytes(self.code, N, D)
            self.bwd_ws = self.L.atexn_layer_norm_bwd_workspace_bytes(self.code, N, D)
        else:
            N, C, D, cf = dims
            shape, stat_shape, P = ((N, C, D) if cf else (N, D, C)), (N, C), C
            self.layout = 0 if cf else 1
            self.fwd_ws = self.L.atexn_instance_norm_fwd_workspace_bytes(self.code, self.layout, N, C, D)
            self.bwd_ws = self.L.atexn_instance_norm_bwd_workspace_bytes(self.code, self.layout, N, C, D)
        n_elem = int(np.prod(shape))
        set_bytes = 4 * n_elem * ESIZE[dtype]
        self.n_sets = max(2, min(64, -(-ROTATE_BYTES // set_bytes)))
        g = torch.Generator(device=device)
        g.manual_seed(1234)
        self.sets = []
        for _ in range(self.n_sets):
            x = (torch.randn(shape, device=device, dtype=torch.float32, generator=g)).to(tdt)
            dy = torch.randn(shape, device=device, dtype=torch.float32, generator=g).to(tdt)
            self.sets.append(dict(
                x=x, dy=dy, y=torch.empty_like(x), dx=torch.empty_like(x),
                mean=torch.empty(stat_shape, device=device, dtype=torch.float32),
                rstd=torch.empty(stat_shape, device=device, dtype=torch.float32)))
        self.gamma = torch.rand(P, device=device, dtype=torch.float32, generator=g) + 0.5
        self.beta = torch.randn(P, device=device, dtype=torch.float32, generator=g) * 0.1
        self.dgamma = torch.empty(P, device=device, dtype=torch.float32)
        self.dbeta = torch.empty(P, device=device, dtype=torch.float32)
        wsb = max(self.fwd_ws, self.bwd_ws, 256)
        self.ws = torch.empty(wsb, device=device, dtype=torch.uint8)
        self.stream = torch.cuda.current_stream(device).cuda_stream

    def fwd(self, i):
        s = self.sets[i % self.n_sets]
        L, c = self.L, self.code
        if self.op == "ln":
            N, D = self.dims
            st = L.atexn_layer_norm_fwd(c, s["x"].data_ptr(), self.gamma.data_ptr(), self.beta.data_ptr(), N, D,
                                        1e-3, s["y"].data_ptr(), s["mean"].data_ptr(), s["rstd"].data_ptr(),
                                        self.ws.data_ptr(), self.ws.numel(), self.stream)
        else:
            N, C, D, _ = self.dims
            st = L.atexn_instance_norm_fwd(c, self.layout, s["x"].data_ptr(), self.gamma.data_ptr(),
                                           self.beta.data_ptr(), N, C, D, 1e-3, s["y"].data_ptr(),
                                           s["mean"].data_ptr(), s["rstd"].data_ptr(), self.ws.data_ptr(),
                                           self.ws.numel(), self.stream)
        if st != 0:
            self.capi.check(st, self.L)

    def bwd(self, i):
        s = self.sets[i % self.n_sets]
        L, c = self.L, self.code
        if self.op == "ln":
            N, D = self.dims
            st = L.atexn_layer_norm_bwd(c, s["dy"].data_ptr(), s["x"].data_ptr(), self.gamma.data_ptr(),
                                        s["mean"].data_ptr(), s["rstd"].data_ptr(), N, D, s["dx"].data_ptr(),
                                        self.dgamma.data_ptr(), self.dbeta.data_ptr(), self.ws.data_ptr(),
                                        self.ws.numel(), self.stream)
        else:
            N, C, D, _ = self.dims
            st = L.atexn_instance_norm_bwd(c, self.layout, s["dy"].data_ptr(), s["x"].data_ptr(),
                                           self.gamma.data_ptr(), s["mean"].data_ptr(), s["rstd"].data_ptr(),
                                           N, C, D, s["dx"].data_ptr(), self.dgamma.data_ptr(),
                                           self.dbeta.data_ptr(), self.ws.data_ptr(), self.ws.numel(), self.stream)
        if st != 0:
            self.capi.check(st, self.L)

    def time_loop(self, fn, steps, warmup):
        """Average milliseconds per call of fn(i), events on the launch stream."""
        torch = self.torch
        for i in range(warmup):
            fn(i)
        torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        for i in range(steps):
            fn(warmup + i)
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / steps


def cpu_baseline(op, dtype, dims, max_seconds=20.0):
    """The oracle's float flavour on the same workload (full size when it fits the time
    bound, else the leading rows / instances), OpenMP threads = host cores in use."""
    from oracle import oracle as O

    O.build()
    co = O.COracle()
    threads = min(16, os.cpu_count() or 1)
    co.set_num_threads(threads)
    sample = "full workload"
    d = list(dims)
    if op == "in" and d[2] * d[1] * d[0] > 32 * 1024 * 1024:
        d[0] = 1
        sample = f"first instance only (N=1 of {dims[0]})"
    d = tuple(d)
    x, gamma, beta, dy = make_host_inputs(op, dtype, d, 1001)
    xs, dys = _storage(x, dtype), _storage(dy, dtype)

    def step():
        if op == "ln":
            y, m, r = co.ln_fwd(xs, gamma, beta, 1e-3, dtype, f64=False)
            co.ln_bwd(dys, xs, gamma, m, r, dtype, f64=False)
        else:
            cf = d[3]
            y, m, r = co.in_fwd(xs, gamma, beta, 1e-3, dtype, cf, f64=False)
            co.in_bwd(dys, xs, gamma, m, r, dtype, cf, f64=False)

    step()
    times = []
    t_end = time.perf_counter() + max_seconds
    while len(times) < 10 and (time.perf_counter() < t_end or len(times) < 2):
        t0 = time.perf_counter()
        step()
        times.append(time.perf_counter() - t0)
    med = float(np.median(times))
    fb, bb = algorithmic_bytes(op, dtype, d)
    return {
        "value": (fb + bb) / med / 1e9,
        "unit": "GB/s",
        "cores": threads,
        "kind": "port",
        "sample": f"{sample}; median of {len(times)} steps, {med * 1e6:.0f} us/step",
        "us_per_step": med * 1e6,
        "unfused_composite": composite_cpu(op, dtype, d, x, gamma, beta, dy, threads),
    }


def composite_cpu(op, dtype, d, x, gamma, beta, dy, threads, max_seconds=8.0):
    """What a framework without the fused op runs on the host: the unfused op sequence
    (moments -> subtract -> rsqrt -> multiply -> add, statistics in float32, autograd for
    the backward) in torch on the CPU.  A composite restatement, not tf.keras itself
    (TensorFlow is not installed); reported beside the fused C port for orientation."""
    import torch

    torch.set_num_threads(threads)
    tdt = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[dtype]
    xt = torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).to(tdt).requires_grad_(True)
    g = torch.from_numpy(gamma).requires_grad_(True)
    b = torch.from_numpy(beta).requires_grad_(True)
    dyt = torch.from_numpy(np.ascontiguousarray(dy, dtype=np.float32)).to(tdt)
    if op == "ln":
        axes, wshape = (-1,), (1, -1)
    elif d[3]:   # channel-first [N, C, D]
        axes, wshape = (2,), (1, -1, 1)
    else:        # channels-last [N, D, C]
        axes, wshape = (1,), (1, 1, -1)

    def step():
        xf = xt.float()
        mean = xf.mean(dim=axes, keepdim=True)
        var = (xf - mean).square().mean(dim=axes, keepdim=True)
        y = ((xf - mean) * torch.rsqrt(var + 1e-3) * g.view(wshape) + b.view(wshape)).to(tdt)
        torch.autograd.grad(y, (xt, g, b), dyt)

    step()
    times = []
    t_end = time.perf_counter() + max_seconds
    while len(times) < 10 and (time.perf_counter() < t_end or len(times) < 2):
        t0 = time.perf_counter()
        step()
        times.append(time.perf_counter() - t0)
    med = float(np.median(times))
    fb, bb = algorithmic_bytes(op, dtype, d)
    return {"value": (fb + bb) / med / 1e9, "unit": "GB/s", "threads": threads,
            "us_per_step": med * 1e6,
            "note": "torch CPU, unfused op sequence with autograd; composite restatement, not tf.keras"}


def describe_bwd(op, dtype, dims):
    """(text, alone): the kernels the backward of the case launches, from the library's own
    planner (benchmark build), and whether its row kernel can be timed without the column
    reduction that follows it."""
    import ctypes

    LB = bench_lib()
    if LB is None:
        return "backward call (benchmark build of the library missing: no plan description)", False
    buf = ctypes.create_string_buffer(512)
    code = {"f32": 0, "f16": 1, "bf16": 2}[dtype]
    if op == "ln":
        n = LB.atexn_bench_describe_bwd(0, code, 0, dims[0], 0, dims[1], buf, 512)
    else:
        N, C, D, cf = dims
        n = LB.atexn_bench_describe_bwd(1, code, 0 if cf else 1, N, C, D, buf, 512)
    text = buf.value.decode() if n > 0 else "backward call"
    plan, _, alone = text.partition("; alone=")
    return plan, alone == "1"


def torch_mod():
    import torch

    return torch


def time_row_kernel_alone(case, steps, warmup):
    """Average ms of the backward call without its final column reduction (the dominant kernel
    alone), through the benchmark build of the library; None if that build is missing or the
    case's backward has no separate column reduction to switch off."""
    if not describe_bwd(case.op, case.dtype, case.dims)[1]:
        return None
    LB = bench_lib()
    if LB is None:
        return None
    product = case.L
    case.L = LB
    try:
        if LB.atexn_set_tuning(b"bwd_stage_mask", 1) != 0:
            return None
        try:
            return case.time_loop(case.bwd, steps, warmup)
        finally:
            LB.atexn_set_tuning(b"bwd_stage_mask", 3)
    finally:
        case.L = product


def measure(name, steps, warmup, extras=True, streaming=True):
    """Times one case; returns (result dict, GpuCase).  extras: the hot-cache and HIP-graph
    legs; streaming: torch's copy / add on the same tensors."""
    op, dtype, dims = CASES[name]
    fb, bb = algorithmic_bytes(op, dtype, dims)
    case = GpuCase(op, dtype, dims)

    def step(i):
        case.fwd(i)
        case.bwd(i)

    ms_step = case.time_loop(step, steps, warmup)
    ms_fwd = case.time_loop(case.fwd, steps, warmup)
    ms_bwd = case.time_loop(case.bwd, steps, warmup)
    ms_alone = time_row_kernel_alone(case, steps, warmup)
    ms_roof = ms_alone if ms_alone is not None else ms_bwd
    achieved = bb / (ms_roof * 1e-3) / 1e9
    value = (fb + bb) / (ms_step * 1e-3) / 1e9
    if op == "ln":
        workload = f"LayerNorm fwd+bwd x {dtype} [{dims[0]},{dims[1]}] axis=-1 eps=1e-3, gamma/beta fp32"
    else:
        N, C, D, cf = dims
        workload = (f"InstanceNorm fwd+bwd x {dtype} N={N} C={C} spatial={D} "
                    f"{'channel-first' if cf else 'channels-last'} eps=1e-3")
    res = {
        "workload": workload, "case": name, "rotating_buffer_sets": case.n_sets,
        "algorithmic_bytes_fwd": fb, "algorithmic_bytes_bwd": bb,
        "value": value, "ms_per_step": ms_step,
        "pct_of_hbm_peak": 100.0 * value / HBM_PEAK_GBPS,
        "us_per_call": {"fwd": ms_fwd * 1e3, "bwd": ms_bwd * 1e3, "fwd_bwd": ms_step * 1e3},
        "gbps": {"fwd": fb / (ms_fwd * 1e-3) / 1e9, "bwd": bb / (ms_bwd * 1e-3) / 1e9},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBPS, "traffic": MEASURED_TRAFFIC.get(name),
                     "kernel": describe_bwd(op, dtype, dims)[0] +
                               (": the row kernel timed alone, without col_reduce" if ms_alone is not None
                                else ": the whole backward call"),
                     "us": ms_roof * 1e3},
    }
    if streaming:
        res["streaming_reference"] = streaming_reference(case, steps, warmup)
    if not extras:
        return res, case

    # hot-cache figure (one buffer set reused), labelled as such
    n_sets = case.n_sets
    case.n_sets = 1
    ms_step_hot = case.time_loop(step, steps, warmup)
    case.n_sets = n_sets
    res["us_per_call"]["fwd_bwd_hot_cache"] = ms_step_hot * 1e3
    res["gbps"]["fwd_bwd_hot_cache"] = (fb + bb) / (ms_step_hot * 1e-3) / 1e9

    # the same fwd + bwd steps captured once into a HIP graph (one pass over all buffer sets)
    # and replayed: what a caller that captures its step gets
    ms_step_graph = None
    try:
        side = torch_mod().cuda.Stream()
        side.wait_stream(torch_mod().cuda.current_stream())
        graph = torch_mod().cuda.CUDAGraph()
        with torch_mod().cuda.stream(side):
            old = case.stream
            case.stream = side.cuda_stream
            step(0)
            side.synchronize()
            with torch_mod().cuda.graph(graph, stream=side):
                for i in range(case.n_sets):
                    step(i)
            case.stream = old
        torch_mod().cuda.synchronize()
        reps = max(1, steps // case.n_sets)
        ms_step_graph = case.time_loop(lambda i: graph.replay(), reps, 2) / case.n_sets
    except Exception as e:  # graph capture is an extra, never fatal
        print(f"hip graph timing skipped: {e}", file=sys.stderr)
    res["us_per_call"]["fwd_bwd_hip_graph"] = None if ms_step_graph is None else ms_step_graph * 1e3

    return res, case


def streaming_reference(case, steps, warmup):
    """What plain streaming kernels reach on the same tensors and rotation (torch's elementwise
    kernels): a copy (1 read + 1 write, the forward's traffic) and an add (2 reads + 1 write,
    the backward's)."""
    torch = case.torch
    tensor_bytes = case.sets[0]["x"].numel() * ESIZE[case.dtype]
    ms_copy = case.time_loop(lambda i: case.sets[i % case.n_sets]["y"].copy_(case.sets[i % case.n_sets]["x"]),
                             steps, warmup)
    ms_add = case.time_loop(lambda i: torch.add(case.sets[i % case.n_sets]["x"], case.sets[i % case.n_sets]["dy"],
                                                out=case.sets[i % case.n_sets]["dx"]), steps, warmup)
    return {
        "copy_us": ms_copy * 1e3, "copy_gbps": 2 * tensor_bytes / (ms_copy * 1e-3) / 1e9,
        "add_us": ms_add * 1e3, "add_gbps": 3 * tensor_bytes / (ms_add * 1e-3) / 1e9,
        "note": "torch elementwise copy (1r+1w) and add (2r+1w) on the same rotating tensors"}


def torch_ops_reference(case, steps, warmup):
    """What the stock PyTorch-ROCm operators take on the same tensors and rotation: aten's
    native_layer_norm / native_group_norm(groups = C) and their backward operators, called
    directly (no autograd graph), event-timed like the library's calls.  gamma / beta are cast to
    the storage dtype, which those operators require.  Channels-last InstanceNorm has no aten
    kernel (group_norm wants channel-first memory), so that layout reports None."""
    torch = case.torch
    if case.op == "in" and case.layout == 1:
        return None
    tdt = case.sets[0]["x"].dtype
    gamma, beta = case.gamma.to(tdt), case.beta.to(tdt)
    try:
        if case.op == "ln":
            N, D = case.dims
            fwd = lambda i: torch.native_layer_norm(case.sets[i % case.n_sets]["x"], [D], gamma, beta, 1e-3)
            _, mean, rstd = fwd(0)
            bwd = lambda i: torch.ops.aten.native_layer_norm_backward(
                case.sets[i % case.n_sets]["dy"], case.sets[i % case.n_sets]["x"], [D], mean, rstd, gamma, beta,
                [True, True, True])
        else:
            N, C, D, _ = case.dims
            fwd = lambda i: torch.native_group_norm(case.sets[i % case.n_sets]["x"], gamma, beta, N, C, D, C, 1e-3)
            _, mean, rstd = fwd(0)
            bwd = lambda i: torch.ops.aten.native_group_norm_backward(
                case.sets[i % case.n_sets]["dy"], case.sets[i % case.n_sets]["x"], mean, rstd, gamma, N, C, D, C,
                [True, True, True])

        def step(i):
            fwd(i)
            bwd(i)

        ms_step = case.time_loop(step, steps, warmup)
        ms_fwd = case.time_loop(fwd, steps, warmup)
        ms_bwd = case.time_loop(bwd, steps, warmup)
    except Exception as e:  # a comparison, never fatal
        return {"error": str(e)[:200]}
    return {"fwd_us": ms_fwd * 1e3, "bwd_us": ms_bwd * 1e3, "fwd_bwd_us": ms_step * 1e3,
            "note": "aten native_layer_norm / native_group_norm(groups=C) and their backward operators, "
                    "PyTorch-ROCm as installed, same rotating tensors"}


def shared_gpu_reference(name, occupier_wgs=128, hold_ms=20.0, reps=7):
    """One InstanceNorm case beside a kernel that holds whole CUs (atexn_bench_occupy of the
    benchmark build, on a second stream, started first): single forward and backward calls, with
    the kernels whose workgroups exchange results and with the two-launch kernels.  The first
    exchange call pays for waits that run out; the later ones give such waits up early."""
    global USE_BENCH_LIB_EVERYWHERE
    op, dtype, dims = CASES[name]
    if op != "in":
        return None
    torch = torch_mod()
    L = bench_lib()
    if L is None:
        return {"error": "needs the benchmark build of the library"}
    saved = USE_BENCH_LIB_EVERYWHERE
    USE_BENCH_LIB_EVERYWHERE = True
    out = {"occupier": f"{occupier_wgs} workgroups x 1024 threads x 158 KB of LDS, held for {hold_ms:g} ms on a second stream"}
    try:
        case = GpuCase(op, dtype, dims)
        side = torch.cuda.Stream()

        def one(fn, i):
            torch.cuda.synchronize()
            if L.atexn_bench_occupy(occupier_wgs, hold_ms, side.cuda_stream) != 0:
                raise RuntimeError(L.atexn_last_error().decode())
            torch.cuda._sleep(400000)  # the occupier gets its CUs first
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            fn(i)
            e1.record()
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) * 1e3

        for knob, label in ((1, "exchange"), (0, "two_launch")):
            for nm in (b"cl_single", b"plane_single", b"affine_fold"):
                L.atexn_set_tuning(nm, knob)
            L.atexn_bench_mark_exchange_trouble(0)
            case.fwd(0)
            case.bwd(0)
            f = [one(case.fwd, i) for i in range(reps)]
            L.atexn_bench_mark_exchange_trouble(0)
            b = [one(case.bwd, i) for i in range(reps)]
            out[label] = {"fwd_first_us": f[0], "fwd_us": float(np.median(f[1:])),
                          "bwd_first_us": b[0], "bwd_us": float(np.median(b[1:]))}
        del case
    finally:
        for nm in (b"cl_single", b"plane_single", b"affine_fold"):
            L.atexn_set_tuning(nm, 1)
        L.atexn_bench_mark_exchange_trouble(0)
        USE_BENCH_LIB_EVERYWHERE = saved
    return out


# the benchmark configurations beside the default case and the targets, on the default run's line
CONFIG_CASES = ("ln_cfg0", "ln_128_f16", "ln_128_bf16", "ln_4096_f16", "ln_4096_bf16", "ln_12288_f16",
                "ln_12288_bf16", "in3d_ndhwc", "in3d_ncdhw")


def steps_for(name, steps):
    """Fewer timed steps for the 268 MB-per-tensor volumes (a step there is a third of a millisecond)."""
    return max(10, steps // 10) if "3d" in name else steps


def run_case(name, steps, warmup, with_cpu=True, with_targets=False, cold_only=False, torch_ops=False,
             shared_gpu=0):
    op, dtype, dims = CASES[name]
    m, case = measure(name, steps, warmup, extras=not cold_only)
    if torch_ops:
        m["torch_ops"] = torch_ops_reference(case, steps, warmup)
    out = {
        "metric": "LN/IN fwd+bwd achieved HBM GB/s",
        "value": m["value"],
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": m["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": dtype,
        "data": "synthetic",
        "config": {"workload": m["workload"], "case": name, "rotating_buffer_sets": m["rotating_buffer_sets"],
                   "algorithmic_bytes_fwd": m["algorithmic_bytes_fwd"],
                   "algorithmic_bytes_bwd": m["algorithmic_bytes_bwd"]},
        "pct_of_hbm_peak": m["pct_of_hbm_peak"],
        "us_per_call": m["us_per_call"],
        "gbps": m["gbps"],
        "streaming_reference": m.get("streaming_reference"),
        "roofline": m["roofline"],
    }
    if torch_ops:
        out["torch_ops"] = m["torch_ops"]
    del case
    if shared_gpu:
        torch_mod().cuda.empty_cache()
        out["shared_gpu"] = shared_gpu_reference(name, occupier_wgs=shared_gpu)
    if with_targets:
        # the second target shape, on the same driver-run line
        out["targets"] = {}
        for tname in TARGET_CASES:
            if tname == name:
                continue
            t, tcase = measure(tname, steps, warmup, extras=False, streaming=not cold_only)
            del tcase
            torch_mod().cuda.empty_cache()
            out["targets"][tname] = {
                "workload": t["workload"], "dtype": CASES[tname][1],
                "us_per_call": t["us_per_call"], "gbps": t["gbps"],
                "value": t["value"], "pct_of_hbm_peak": t["pct_of_hbm_peak"],
                "roofline": t["roofline"],
            }
            if "streaming_reference" in t:
                out["targets"][tname]["streaming_reference"] = t["streaming_reference"]
        # every other benchmark configuration
        out["configs"] = {}
        for cname in CONFIG_CASES:
            if cname == name:
                continue
            c, ccase = measure(cname, steps_for(cname, steps), warmup, extras=False, streaming=not cold_only)
            del ccase
            torch_mod().cuda.empty_cache()
            out["configs"][cname] = {k: c[k] for k in ("workload", "us_per_call", "gbps", "value", "pct_of_hbm_peak",
                                                       "roofline", "streaming_reference") if k in c}
            out["configs"][cname]["dtype"] = CASES[cname][1]
            out["configs"][cname]["steps"] = steps_for(cname, steps)
    if with_cpu:
        out["cpu_baseline"] = cpu_baseline(op, dtype, dims)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--case", default=DEFAULT_CASE, choices=sorted(CASES) + ["all"])
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--tune", action="append", default=[], metavar="NAME=VALUE",
                    help="set a launch-planning parameter (atexn_set_tuning) before measuring, "
                         "in the product and the benchmark build of the library; for A/B runs")
    ap.add_argument("--no-targets", action="store_true",
                    help="default case only: skip the InstanceNorm target shapes and the other configurations")
    ap.add_argument("--cold-only", action="store_true",
                    help="only the rotating-buffer (cold) legs: no hot-cache loop and no HIP-graph replay (and no "
                         "torch copy / add for the targets and configurations of the default run); what a "
                         "rocprofv3 kernel trace of this file should average over")
    ap.add_argument("--torch-ops", action="store_true",
                    help="also time PyTorch-ROCm's own layer_norm / group_norm(groups=C) operators, forward and "
                         "backward, on the same tensors (the case itself only, not the targets / configurations)")
    ap.add_argument("--shared-gpu", type=int, default=0, metavar="WORKGROUPS",
                    help="InstanceNorm cases: also time single calls while a busy kernel of the benchmark build "
                         "holds that many whole CUs on a second stream (e.g. 128: half the chip)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="after the case, run 5 elementwise negations of a 64 MiB tensor into "
                         "another (torch's neg kernel: reads 64 MiB, writes 64 MiB): a kernel of "
                         "known traffic that scales the FETCH_SIZE / WRITE_SIZE counters of a "
                         "rocprofv3 --pmc run")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: the path has no cross-GPU exchange; run with --gpus 1")
    import torch

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU (no CPU fallback exists for the product path)")
    for item in args.tune:
        global USE_BENCH_LIB_EVERYWHERE
        USE_BENCH_LIB_EVERYWHERE = True
        key, _, val = item.partition("=")
        L = bench_lib()
        if L is None:
            sys.exit("--tune needs the benchmark build of the library (python -m atex_amd.build)")
        if L.atexn_set_tuning(key.encode(), int(val)) != 0:
            sys.exit(f"--tune {item}: {L.atexn_last_error().decode()}")
    if args.case == "all":
        for name in CASES:
            if name in SWEEP_ONLY_CASES:
                continue
            r = run_case(name, steps_for(name, args.steps), args.warmup, with_cpu=False, cold_only=args.cold_only,
                         torch_ops=args.torch_ops, shared_gpu=args.shared_gpu)
            print(json.dumps(r), flush=True)
        return
    print(json.dumps(run_case(args.case, args.steps, args.warmup, with_cpu=not args.no_cpu,
                              with_targets=args.case == DEFAULT_CASE and not args.no_targets,
                              cold_only=args.cold_only, torch_ops=args.torch_ops,
                              shared_gpu=args.shared_gpu)), flush=True)
    if args.copy_calibration:
        src = torch.randn(32 << 20, device="cuda:0", dtype=torch.float16)  # 64 MiB
        dst = torch.empty_like(src)
        for _ in range(5):
            torch.neg(src, out=dst)
        torch.cuda.synchronize()


if __name__ == "__main__":
    main()
