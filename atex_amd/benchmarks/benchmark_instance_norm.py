"""InstanceNorm (3-D volumes) forward + backward, milliseconds per train step, on the shape
table of the reference's benchmark (benchmark_instance_norm.py:58-69), both layouts, fp16
activations with float32 weights.

    python -m atex_amd.benchmarks.benchmark_instance_norm [--json FILE]

Columns: torch's group_norm with one group per channel on the same GPU (the role
tensorflow_addons plays in the reference's table; channels-last inputs are handed to it as a
permuted view, which is what a torch user would do), this library's InstanceNormalization
layer, and the reference's published A100 / H100 figures for its fused op
(README.md:62-108 of atex/nv_norms), for orientation only.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F

from atex_amd import nv_norms
from atex_amd.benchmarks.common import REPEAT, WARMUP, fmt, one_step_outputs, time_train_step, write_json

# (N, C, spatial extent) -> ((A100, H100) channels-last, (A100, H100) channel-first)
SHAPES = {
    (2, 32, 6): ((0.78, 0.70), (0.77, 0.69)),
    (2, 32, 128): ((7.51, 6.05), (5.20, 3.85)),
    (2, 64, 128): ((12.53, 8.69), (10.53, 7.57)),
    (4, 32, 128): ((12.35, 8.70), (9.27, 6.16)),
    (4, 64, 64): ((5.36, 4.63), (2.98, 2.17)),
    (8, 32, 64): ((5.35, 4.66), (3.01, 2.17)),
    (8, 64, 64): ((7.65, 5.98), (5.32, 3.51)),
    (8, 128, 64): ((12.33, 8.63), (10.37, 6.38)),
    (4, 256, 32): ((3.76, 3.57), (1.18, 0.91)),
    (8, 256, 32): ((5.01, 4.25), (2.57, 1.71)),
}


def expand(s, channel_last):
    n, c, d = s
    return (n, d, d, d, c) if channel_last else (n, c, d, d, d)


def _case(shape, channel_last: bool, use_fused: bool):
    """(x, fn, params) of one column of the table."""
    torch.manual_seed(0)
    x = torch.randn(shape, device="cuda", dtype=torch.float16, requires_grad=True)
    c = shape[-1] if channel_last else shape[1]
    if use_fused:
        layer = nv_norms.InstanceNormalization(axis=-1 if channel_last else 1)
        layer.build(shape, device="cuda")
        return x, layer, [layer.gamma, layer.beta]
    gamma = torch.ones(c, device="cuda", requires_grad=True)
    beta = torch.zeros(c, device="cuda", requires_grad=True)
    if channel_last:
        fn = lambda t: F.group_norm(t.permute(0, 4, 1, 2, 3), c, gamma.half(), beta.half(), 1e-3).permute(0, 2, 3, 4, 1)  # noqa: E731
    else:
        fn = lambda t: F.group_norm(t, c, gamma.half(), beta.half(), 1e-3)  # noqa: E731
    return x, fn, [gamma, beta]


def benchmark(shape, channel_last: bool, use_fused: bool, warmup: int = WARMUP, repeat: int = REPEAT) -> float:
    x, fn, params = _case(shape, channel_last, use_fused)
    return time_train_step(x, fn, params, warmup, repeat)


def outputs(shape, channel_last: bool, use_fused: bool):
    """(y, dx, dgamma, dbeta) of one train step of a column."""
    return one_step_outputs(*_case(shape, channel_last, use_fused))


def run(shapes=None, warmup: int = WARMUP, repeat: int = REPEAT, echo=None):
    rows = []
    for channel_last in (True, False):
        for s, pub in SHAPES.items():
            if shapes is not None and s not in shapes:
                continue
            shape = expand(s, channel_last)
            a100, h100 = pub[0] if channel_last else pub[1]
            row = {"shape": list(shape), "layout": "channels_last" if channel_last else "channels_first",
                   "torch_ms": benchmark(shape, channel_last, False, warmup, repeat),
                   "fused_ms": benchmark(shape, channel_last, True, warmup, repeat),
                   "a100_nv_ms": a100, "h100_nv_ms": h100}
            rows.append(row)
            if echo:
                echo(row)
    return rows


def main():
    import argparse

    ap = argparse.ArgumentParser()
    ap.add_argument("--json", metavar="FILE", help="also write the table as JSON")
    args = ap.parse_args()
    if not torch.cuda.is_available():
        raise SystemExit("needs a GPU")
    print("InstanceNorm fwd+bwd, fp16, ms per train step; channels_last (N, D, H, W, C) then channels_first (N, C, D, H, W)")
    print(f"{'shape':>24} | {'torch':>7} {'fused':>7} | A100 NV  H100 NV (published, other hardware)")
    rows = run(echo=lambda r: print(f"{str(tuple(r['shape'])):>24} | {r['torch_ms']:7.3f} {r['fused_ms']:7.3f} | "
                                    f"{fmt(r['a100_nv_ms'])}   {fmt(r['h100_nv_ms'])}", flush=True))
    if args.json:
        write_json(args.json, "InstanceNorm 3-D volumes, fp16 activations, float32 weights", rows)


if __name__ == "__main__":
    main()
