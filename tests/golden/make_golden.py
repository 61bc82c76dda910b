#!/usr/bin/env python3
"""Writes the golden fixtures tests/golden/*.npz.

The reference ships no golden vectors (its tests draw unseeded random inputs and compare with
tf.keras / tensorflow_addons on a GPU), and neither TensorFlow nor the reference's own code
can run in this environment.  These fixtures are therefore produced by an INDEPENDENT
third-party implementation of the same mathematics that is available here: torch's CPU
float64 `native_layer_norm` / `group_norm` (groups = C is instance normalisation) for the
forward pass and torch autograd through them for the backward pass.  Nothing under oracle/
or atex_amd/ is imported: the fixtures pin the oracle and the HIP kernels, not vice versa.

Inputs are seeded (numpy PCG64) and rounded to the storage dtype before the float64
evaluation, so that every implementation sees identical values.  To keep the files small,
x / dy are stored in the storage dtype (bfloat16 as uint16 bit patterns), y / dx as float32
(the float64 result rounded once) and the statistics and parameter gradients as float64.

    python tests/golden/make_golden.py
"""
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
EPS = 1e-3


def rng_for(i):
    return np.random.Generator(np.random.PCG64(7000 + i))


def round_to(a, dtype):
    """float32 values rounded to the storage dtype, returned as float32 (exactly representable)."""
    t = torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32))
    if dtype == "f16":
        t = t.to(torch.float16).to(torch.float32)
    elif dtype == "bf16":
        t = t.to(torch.bfloat16).to(torch.float32)
    return t.numpy()


def store(a, dtype):
    """float32 values that are exact in `dtype` -> the dtype's in-memory representation."""
    t = torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32))
    if dtype == "f16":
        return t.to(torch.float16).numpy()
    if dtype == "bf16":
        return t.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    return t.numpy()


def ln_case(idx, N, D, dtype, loc=0.0, scale=1.0):
    r = rng_for(idx)
    x = round_to(r.standard_normal((N, D)) * scale + loc, dtype)
    dy = round_to(r.standard_normal((N, D)), dtype)
    gamma = r.uniform(0.5, 1.5, size=D).astype(np.float32)
    beta = (r.standard_normal(D) * 0.1).astype(np.float32)
    xt = torch.from_numpy(x).double().requires_grad_(True)
    gt = torch.from_numpy(gamma).double().requires_grad_(True)
    bt = torch.from_numpy(beta).double().requires_grad_(True)
    y, mean, rstd = torch.native_layer_norm(xt, [D], gt, bt, EPS)
    y.backward(torch.from_numpy(dy).double())
    return dict(kind="ln", dtype=dtype, eps=EPS, x=store(x, dtype), dy=store(dy, dtype), gamma=gamma,
                beta=beta, y=y.detach().numpy().astype(np.float32),
                mean=mean.detach().numpy().reshape(N), inv_std=rstd.detach().numpy().reshape(N),
                dx=xt.grad.numpy().astype(np.float32), dgamma=gt.grad.numpy(), dbeta=bt.grad.numpy())


def in_case(idx, N, C, spatial, dtype, channel_first, loc=0.0, scale=1.0):
    r = rng_for(idx)
    # generated channel-first [N, C, D]; the channels-last variant is the transpose
    x = round_to(r.standard_normal((N, C, spatial)) * scale + loc + r.uniform(-1, 1, size=(1, C, 1)), dtype)
    dy = round_to(r.standard_normal((N, C, spatial)), dtype)
    gamma = r.uniform(0.5, 1.5, size=C).astype(np.float32)
    beta = (r.standard_normal(C) * 0.1).astype(np.float32)
    xt = torch.from_numpy(x).double().requires_grad_(True)
    gt = torch.from_numpy(gamma).double().requires_grad_(True)
    bt = torch.from_numpy(beta).double().requires_grad_(True)
    y = torch.nn.functional.group_norm(xt, C, gt, bt, EPS)
    y.backward(torch.from_numpy(dy).double())
    xd = xt.detach()
    mean = xd.mean(dim=2)
    var = xd.var(dim=2, unbiased=False)
    out = dict(kind="in", dtype=dtype, eps=EPS, channel_first=channel_first, gamma=gamma, beta=beta,
               mean=mean.numpy(), inv_std=(1.0 / torch.sqrt(var + EPS)).numpy(),
               dgamma=gt.grad.numpy(), dbeta=bt.grad.numpy())
    tensors = dict(x=x, dy=dy, y=y.detach().numpy().astype(np.float32),
                   dx=xt.grad.numpy().astype(np.float32))
    for k, v in tensors.items():
        v = v if channel_first else np.ascontiguousarray(np.transpose(v, (0, 2, 1)))
        out[k] = store(v, dtype) if k in ("x", "dy") else v
    return out


CASES = {
    # LayerNorm: lanes-per-row, block-per-row and element-wise kernel families, all dtypes
    "ln_f32_8x1024": lambda: ln_case(0, 8, 1024, "f32"),
    "ln_f16_8x1024": lambda: ln_case(1, 8, 1024, "f16", loc=1.5),
    "ln_bf16_16x128": lambda: ln_case(2, 16, 128, "bf16"),
    "ln_f16_2x4096": lambda: ln_case(3, 2, 4096, "f16"),
    "ln_f32_5x31": lambda: ln_case(4, 5, 31, "f32", scale=10.0),
    "ln_f16_3x2003": lambda: ln_case(5, 3, 2003, "f16", scale=10.0),
    "ln_f32_4x256_large_mean": lambda: ln_case(7, 4, 256, "f32", loc=500.0, scale=280.0),
    # InstanceNorm: both layouts, odd channel counts
    "in_f16_cl_2x16x256": lambda: in_case(10, 2, 16, 256, "f16", False),
    "in_f16_cf_2x16x256": lambda: in_case(11, 2, 16, 256, "f16", True),
    "in_f32_cl_1x5x777": lambda: in_case(12, 1, 5, 777, "f32", False, scale=10.0),
    "in_f32_cf_1x5x777": lambda: in_case(13, 1, 5, 777, "f32", True, scale=10.0),
    "in_bf16_cl_2x64x100": lambda: in_case(14, 2, 64, 100, "bf16", False),
    "in_f32_cf_1x2x9000": lambda: in_case(15, 1, 2, 9000, "f32", True),
    "in_f32_cl_1x8x2000": lambda: in_case(16, 1, 8, 2000, "f32", False, loc=3.0),
}


def main():
    for name, fn in CASES.items():
        d = fn()
        path = os.path.join(HERE, name + ".npz")
        np.savez_compressed(path, **d)
        print(f"{name}: {os.path.getsize(path) / 1024:.0f} KiB")


if __name__ == "__main__":
    main()
