"""Shared pieces of the two toy models: a channels-last 2-D convolution followed by a
normalisation layer, one training step with a sum loss (the model of
atex/nv_norms/examples/sample_layerN.py:15-44 and sample_instanceN.py:16-46, hosted on torch
because TensorFlow is not part of this stack)."""
from __future__ import annotations

import torch


class ChannelsLastConv2D(torch.nn.Module):
    """Conv2D(filters, (r, s), padding='same') on [N, H, W, C] activations."""

    def __init__(self, in_channels: int, filters: int, kernel=(2, 2)):
        super().__init__()
        self.conv = torch.nn.Conv2d(in_channels, filters, kernel, padding="same")

    def forward(self, x):
        y = self.conv(x.permute(0, 3, 1, 2))
        return y.permute(0, 2, 3, 1).contiguous()


class ToyModel(torch.nn.Module):
    def __init__(self, in_channels: int, filters: int, norm: torch.nn.Module):
        super().__init__()
        self.conv2d = ChannelsLastConv2D(in_channels, filters)
        self.norm = norm

    def forward(self, x):
        return self.norm(self.conv2d(x))


def train_step(model: torch.nn.Module, x: torch.Tensor):
    """loss = sum(model(x)); returns the gradients of every parameter, in
    `model.named_parameters()` order, as a dict."""
    params = dict(model.named_parameters())
    loss = model(x).sum()
    grads = torch.autograd.grad(loss, list(params.values()), allow_unused=True)
    return {k: g for k, g in zip(params, grads)}
