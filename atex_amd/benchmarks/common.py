"""Timing protocol shared by the two benchmark scripts: the reference's train step
(benchmark_layer_norm.py:16-51): forward through the layer, loss = sum(y), gradients with
respect to x, gamma and beta; 10 warm-up steps, 20 timed steps, one host synchronisation at
the end; result in milliseconds per step, eager dispatch overhead included."""
from __future__ import annotations

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
    start = time.perf_counter()
    for _ in range(repeat):
        g = train_step(x, fn, params)
    _ = float(g[0].float().sum())
    return 1000.0 * (time.perf_counter() - start) / repeat


def fmt(v):
    return "   -  " if v is None else f"{v:6.2f}"
