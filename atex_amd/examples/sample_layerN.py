"""Toy model: Conv2D -> LayerNormalization over (H, W, C), one training step.
`--nvops` swaps the framework's layer norm for the fused layer, as the reference's example
does (atex/nv_norms/examples/sample_layerN.py:9-22).

    python -m atex_amd.examples.sample_layerN [--nvops]
"""
from __future__ import annotations

import argparse

import torch

from .toy import ToyModel, train_step

N, H, W, C = 10, 3, 3, 4
FILTERS = 4


class _TorchLayerNorm(torch.nn.Module):
    """torch's own layer norm over the last three dims, epsilon as Keras' default."""

    def __init__(self, shape):
        super().__init__()
        self.inner = torch.nn.LayerNorm(shape, eps=1e-3)

    def forward(self, x):
        return self.inner(x)


def build_model(use_nv_norms: bool, device="cuda") -> ToyModel:
    if use_nv_norms:
        from atex_amd import nv_norms
        norm = nv_norms.LayerNormalization(axis=(1, 2, 3))
        norm.build((N, H, W, FILTERS), device=device)
    else:
        norm = _TorchLayerNorm((H, W, FILTERS))
    return ToyModel(C, FILTERS, norm).to(device)


def main(argv=None):
    parser = argparse.ArgumentParser(description="Use --nvops to replace the layer norm")
    parser.add_argument("--nvops", action="store_true", help="use the fused layer norm")
    args, _ = parser.parse_known_args(argv)
    torch.manual_seed(0)
    model = build_model(args.nvops)
    data = torch.randn(N, H, W, C, device="cuda")
    grads = train_step(model, data)
    next(iter(grads.values())).cpu()  # wait for the GPU
    print("Done with", "Fused LayerN" if args.nvops else "torch LayerN")
    return grads


if __name__ == "__main__":
    main()
