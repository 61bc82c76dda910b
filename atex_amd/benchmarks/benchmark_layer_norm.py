"""LayerNorm forward + backward, milliseconds per train step, on the shape table of the
reference's benchmark (benchmark_layer_norm.py:53-63), fp16 activations with float32 weights
(its mixed_float16 policy).

    python -m atex_amd.benchmarks.benchmark_layer_norm [--json FILE]

Columns: torch's own layer_norm on the same GPU (the role tf.keras plays in the reference's
table), this library's LayerNormalization layer, and the reference's published figures for
its fused op on A100 / H100 (README.md:35-55 of atex/nv_norms) for orientation only: other
hardware, TensorFlow eager overhead included.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F

from atex_amd import nv_norms
from atex_amd.benchmarks.common import REPEAT, WARMUP, fmt, one_step_outputs, time_train_step, write_json

# shape -> (A100 NV, H100 NV) ms per step as published
SHAPES = {
    (10, 10000000): (3.36, 2.36),
    (100, 1000000): (2.78, 1.78),
    (1000, 100000): (2.81, 1.95),
    (10000, 10000): (4.50, 5.84),
    (100000, 1000): (4.32, 4.73),
    (1000000, 100): (6.33, 6.26),
    (10000000, 10): (13.82, 10.61),
    (4, 400001): (0.59, 0.74),  # non-typical shapes
    (4, 10000001): (1.69, 1.15),
}


def _case(shape, use_fused: bool):
    """(x, fn, params) of one column of the table."""
    torch.manual_seed(0)
    x = torch.randn(shape, device="cuda", dtype=torch.float16, requires_grad=True)
    if use_fused:
        layer = nv_norms.LayerNormalization(axis=(1,))
        layer.build(shape, device="cuda")
        return x, layer, [layer.gamma, layer.beta]
    gamma = torch.ones(shape[1], device="cuda", requires_grad=True)
    beta = torch.zeros(shape[1], device="cuda", requires_grad=True)
    # autocast-free mixed precision: float32 weights cast at the call, as torch users do
    fn = lambda t: F.layer_norm(t, (shape[1],), gamma.half(), beta.half(), 1e-3)  # noqa: E731
    return x, fn, [gamma, beta]


def benchmark(shape, use_fused: bool, warmup: int = WARMUP, repeat: int = REPEAT) -> float:
    x, fn, params = _case(shape, use_fused)
    return time_train_step(x, fn, params, warmup, repeat)


def outputs(shape, use_fused: bool):
    """(y, dx, dgamma, dbeta) of one train step of a column."""
    return one_step_outputs(*_case(shape, use_fused))


def run(shapes=None, warmup: int = WARMUP, repeat: int = REPEAT, echo=None):
    rows = []
    for shape, (a100, h100) in SHAPES.items():
        if shapes is not None and shape not in shapes:
            continue
        row = {"shape": list(shape), "torch_ms": benchmark(shape, False, warmup, repeat),
               "fused_ms": benchmark(shape, True, warmup, repeat), "a100_nv_ms": a100, "h100_nv_ms": h100}
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
    print("LayerNorm fwd+bwd, fp16, ms per train step")
    print(f"{'N':>9} {'D':>9} | {'torch':>7} {'fused':>7} | A100 NV  H100 NV (published, other hardware)")
    rows = run(echo=lambda r: print(f"{r['shape'][0]:>9} {r['shape'][1]:>9} | {r['torch_ms']:7.3f} {r['fused_ms']:7.3f} | "
                                    f"{fmt(r['a100_nv_ms'])}   {fmt(r['h100_nv_ms'])}", flush=True))
    if args.json:
        write_json(args.json, "LayerNorm [N, D], fp16 activations, float32 weights", rows)


if __name__ == "__main__":
    main()
