"""Timing protocol shared by the two benchmark scripts: the reference's train step
(benchmark_layer_norm.py:16-51): forward through the layer, loss = sum(y), gradients with
respect to x, gamma and beta; 10 warm-up steps, 20 timed steps, one host synchronisation at
the end; result in milliseconds per step, eager dispatch overhead included.  Python's cyclic
garbage collector is off during the timed steps, as in the standard library's timeit: a full
collection of a process with torch loaded takes tens of milliseconds and would land on
whichever row of a table happens to cross its threshold."""
from __future__ import annotations

import gc
import time

import torch

WARMUP = 10
REPEAT = 20


def train_step(x, fn, params):
    y = fn(x)
    loss = y.sum()
    grads = torch.autograd.grad(loss, [x] + list(params))
    return grads


def time_train_step(x, fn, params, warmup=WARMUP, repeat=REPEAT) -> float:
    for _ in range(warmup):
        g = train_step(x, fn, params)
    _ = float(g[0].float().sum())  # the reference synchronises through reduce_sum(dx).numpy()
    gc.collect()
    gc_was_on = gc.isenabled()
    gc.disable()
    try:
        start = time.perf_counter()
        for _ in range(repeat):
            g = train_step(x, fn, params)
        _ = float(g[0].float().sum())
        elapsed = time.perf_counter() - start
    finally:
        if gc_was_on:
            gc.enable()
    return 1000.0 * elapsed / repeat


def fmt(v):
    return "   -  " if v is None else f"{v:6.2f}"


def one_step_outputs(x, fn, params):
    """(y, dx, dparams...) of a single step, for comparing two columns of a table.  The loss is
    a fixed random weighting of y rather than the timed step's plain sum: with dy = 1 the scale
    gradient is sum(xhat) = 0 and would compare rounding noise only."""
    y = fn(x)
    g = torch.Generator(device=y.device).manual_seed(1)
    w = torch.randn(y.shape, device=y.device, dtype=torch.float32, generator=g).to(y.dtype)
    grads = torch.autograd.grad((y * w).sum(), [x] + list(params))
    return (y.detach(),) + tuple(g.detach() for g in grads)


def write_json(path, table, rows):
    """rows: list of dicts.  Adds what is needed to read the file on its own."""
    import json

    doc = {
        "table": table,
        "unit": "ms per train step (layer forward, sum loss, gradients of x, gamma, beta; eager)",
        "warmup": WARMUP, "repeat": REPEAT,
        "device": torch.cuda.get_device_name(0) if torch.cuda.is_available() else "cpu",
        "columns": {"torch_ms": "torch's own op on the same GPU", "fused_ms": "this library's layer",
                    "a100_nv_ms / h100_nv_ms": "the reference's published figures for its fused op (other hardware)"},
        "rows": rows,
    }
    with open(path, "w") as f:
        json.dump(doc, f, indent=1)
        f.write("\n")
