"""InstanceNorm (3-D volumes) forward + backward, milliseconds per train step, on the shape
table of the reference's benchmark (benchmark_instance_norm.py:58-69), both layouts, fp16
activations with float32 weights.

    python -m atex_amd.benchmarks.benchmark_instance_norm

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
from atex_amd.benchmarks.common import fmt, time_train_step

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


def benchmark(shape, channel_last: bool, use_fused: bool) -> float:
    torch.manual_seed(0)
    x = torch.randn(shape, device="cuda", dtype=torch.float16, requires_grad=True)
    c = shape[-1] if channel_last else shape[1]
    if use_fused:
        layer = nv_norms.InstanceNormalization(axis=-1 if channel_last else 1)
        layer.build(shape, device="cuda")
        return time_train_step(x, layer, [layer.gamma, layer.beta])
    gamma = torch.ones(c, device="cuda", requires_grad=True)
    beta = torch.zeros(c, device="cuda", requires_grad=True)
    if channel_last:
        fn = lambda t: F.group_norm(t.permute(0, 4, 1, 2, 3), c, gamma.half(), beta.half(), 1e-3)  # noqa: E731
    else:
        fn = lambda t: F.group_norm(t, c, gamma.half(), beta.half(), 1e-3)  # noqa: E731
    return time_train_step(x, fn, [gamma, beta])


def main():
    if not torch.cuda.is_available():
        raise SystemExit("needs a GPU")
    for channel_last in (True, False):
        print(f"InstanceNorm fwd+bwd, fp16, {'channels_last (N, D, H, W, C)' if channel_last else 'channels_first (N, C, D, H, W)'}, ms per train step")
        print(f"{'shape':>24} | {'torch':>7} {'fused':>7} | A100 NV  H100 NV (published, other hardware)")
        for s, pub in SHAPES.items():
            shape = expand(s, channel_last)
            a100, h100 = pub[0] if channel_last else pub[1]
            t_native = benchmark(shape, channel_last, False)
            t_fused = benchmark(shape, channel_last, True)
            print(f"{str(shape):>24} | {t_native:7.3f} {t_fused:7.3f} | {fmt(a100)}   {fmt(h100)}", flush=True)


if __name__ == "__main__":
    main()
