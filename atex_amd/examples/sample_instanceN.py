"""Toy model: Conv2D -> InstanceNormalization over the channel axis, one training step.
`--nvops` swaps the framework's instance norm (a group norm with one group per channel) for
the fused layer, as the reference's example does
(atex/nv_norms/examples/sample_instanceN.py:10-24).

    python -m atex_amd.examples.sample_instanceN [--nvops]
"""
from __future__ import annotations

import argparse

import torch

from .toy import ToyModel, train_step

N, H, W, C = 2, 32, 32, 8
FILTERS = 4


class _TorchInstanceNorm(torch.nn.Module):
    """torch's group norm with groups = channels on channels-last activations."""

    def __init__(self, channels):
        super().__init__()
        self.inner = torch.nn.GroupNorm(channels, channels, eps=1e-3)

    def forward(self, x):
        return self.inner(x.permute(0, 3, 1, 2)).permute(0, 2, 3, 1)


def build_model(use_nv_norms: bool, device="cuda") -> ToyModel:
    if use_nv_norms:
        from atex_amd import nv_norms
        norm = nv_norms.InstanceNormalization(axis=-1)
        norm.build((N, H, W, FILTERS), device=device)
    else:
        norm = _TorchInstanceNorm(FILTERS)
    return ToyModel(C, FILTERS, norm).to(device)


def main(argv=None):
    parser = argparse.ArgumentParser(description="Use --nvops to replace the instance norm")
    parser.add_argument("--nvops", action="store_true", help="use the fused instance norm")
    args, _ = parser.parse_known_args(argv)
    torch.manual_seed(0)
    model = build_model(args.nvops)
    data = torch.randn(N, H, W, C, device="cuda")
    grads = train_step(model, data)
    next(iter(grads.values())).cpu()
    print("Done with", "Fused instanceN" if args.nvops else "torch instanceN")
    return grads


if __name__ == "__main__":
    main()
