"""Layer-level surface, mirroring atex/nv_norms/python/ops/nv_norm_ops.py:27-184.

`LayerNormalization` / `InstanceNormalization` keep the reference layers' contract:
they hold gamma / beta (float32 whatever the activation dtype, nv_norm_ops.py:130-143),
call the fused op in the forward pass and return only `y`; the gradient functions
`_layer_norm_grad` / `_instance_norm_grad` take the op's inputs, its saved outputs 1 and 2
and its attribute, exactly like the reference's registered gradients
(nv_norm_ops.py:27-67).  The host framework here is torch (TensorFlow / Keras /
tensorflow_addons are not available): the layers are torch.nn.Module objects and the
gradient registration is a torch.autograd.Function.
"""
from __future__ import annotations

from typing import Sequence, Union

import torch

from . import ops


class _OpRecord:
    """What a TensorFlow `Operation` exposes to a registered gradient function."""

    def __init__(self, inputs, outputs, attrs):
        self.inputs = inputs
        self.outputs = outputs
        self._attrs = attrs

    def get_attr(self, name):
        return self._attrs[name]


def _layer_norm_grad(op: _OpRecord, *grad):
    """Gradient of fused_layer_norm (reference: nv_norm_ops.py:48-67)."""
    x = op.inputs[0]
    gamma = op.inputs[1]
    a = op.outputs[1]
    b = op.outputs[2]
    dx, dgamma, dbeta = ops.fused_layer_norm_grad_op(grad[0], x, gamma, a, b, axis=op.get_attr("axis"))
    return [dx, dgamma, dbeta]


def _instance_norm_grad(op: _OpRecord, *grad):
    """Gradient of fused_instance_norm (reference: nv_norm_ops.py:27-46)."""
    x = op.inputs[0]
    gamma = op.inputs[1]
    a = op.outputs[1]
    b = op.outputs[2]
    dx, dgamma, dbeta = ops.fused_instance_norm_grad_op(
        grad[0], x, gamma, a, b, data_format=op.get_attr("data_format"))
    return [dx, dgamma, dbeta]


class _FusedLayerNormFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, gamma, beta, axis, epsilon):
        y, mean, inv_std = ops.fused_layer_norm_op(x, gamma, beta, axis=axis, epsilon=epsilon)
        ctx.save_for_backward(x, gamma, mean, inv_std)
        ctx.axis = list(axis)
        ctx.mark_non_differentiable(mean, inv_std)
        return y, mean, inv_std

    @staticmethod
    def backward(ctx, dy, _dmean, _dinv_std):
        x, gamma, mean, inv_std = ctx.saved_tensors
        op = _OpRecord([x, gamma, None], [None, mean, inv_std], {"axis": ctx.axis})
        dx, dgamma, dbeta = _layer_norm_grad(op, dy.contiguous())
        return dx, dgamma, dbeta, None, None


class _FusedInstanceNormFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, gamma, beta, data_format, epsilon):
        y, mean, inv_std = ops.fused_instance_norm_op(x, gamma, beta, data_format=data_format, epsilon=epsilon)
        ctx.save_for_backward(x, gamma, mean, inv_std)
        ctx.data_format = data_format
        ctx.mark_non_differentiable(mean, inv_std)
        return y, mean, inv_std

    @staticmethod
    def backward(ctx, dy, _dmean, _dinv_std):
        x, gamma, mean, inv_std = ctx.saved_tensors
        op = _OpRecord([x, gamma, None], [None, mean, inv_std], {"data_format": ctx.data_format})
        dx, dgamma, dbeta = _instance_norm_grad(op, dy.contiguous())
        return dx, dgamma, dbeta, None, None


def fused_layer_norm(x, gamma, beta, axis=(-1,), epsilon=0.001):
    """Differentiable fused_layer_norm_op: returns (y, mean, inv_std)."""
    return _FusedLayerNormFn.apply(x, gamma, beta, tuple(axis), float(epsilon))


def fused_instance_norm(x, gamma, beta, data_format="N...C", epsilon=0.001):
    """Differentiable fused_instance_norm_op: returns (y, mean, inv_std)."""
    return _FusedInstanceNormFn.apply(x, gamma, beta, data_format, float(epsilon))


class LayerNormalization(torch.nn.Module):
    """Same arguments as tf.keras.layers.LayerNormalization that matter to the fused op
    (`axis`, `epsilon`), except that the axes must be packed and include the last
    dimension.  Output: `y`, same shape as the input (reference: nv_norm_ops.py:69-121).

    Like the Keras layer, weights are created by `build(input_shape)` (called on first
    use) with shape `[input_shape[a] for a in axis]`, gamma = 1, beta = 0, float32.
    """

    def __init__(self, axis: Union[int, Sequence[int]] = -1, epsilon: float = 1e-3, **kwargs):
        super().__init__()
        unsupported = {k: v for k, v in kwargs.items()
                       if k in ("center", "scale") and v is not True}
        if unsupported:
            raise ValueError(f"the fused op always centers and scales; got {unsupported}")
        if isinstance(axis, (list, tuple)):
            self.axis = list(axis)
        elif isinstance(axis, int):
            self.axis = axis
        else:
            raise TypeError(f"Expected an int or a list/tuple of ints for `axis`, got {axis!r}")
        self.epsilon = float(epsilon)
        self.gamma = None
        self.beta = None
        self.built = False

    def build(self, input_shape, device=None):
        ndims = len(input_shape)
        # Keras normalises the axis in build(): ints become lists, negatives wrap
        axis = [self.axis] if isinstance(self.axis, int) else list(self.axis)
        for i, a in enumerate(axis):
            if a < 0:
                axis[i] = ndims + a
        for a in axis:
            if a < 0 or a >= ndims:
                raise ValueError(f"Invalid axis: {a}")
        if len(axis) != len(set(axis)):
            raise ValueError(f"Duplicate axis: {tuple(axis)}")
        self.axis = axis
        shape = [int(input_shape[a]) for a in axis]
        self.gamma = torch.nn.Parameter(torch.ones(shape, dtype=torch.float32, device=device))
        self.beta = torch.nn.Parameter(torch.zeros(shape, dtype=torch.float32, device=device))
        self.built = True

    def forward(self, inputs):
        if not self.built:
            self.build(tuple(inputs.shape), device=inputs.device)
        axis = self.axis
        if isinstance(axis, int):
            axis = [axis]
        if axis != sorted(set(axis)):
            raise ValueError("We only support sorted and unique axis to make sure the weights "
                             "have the same data layout with the keras layers.")
        y, _, _ = fused_layer_norm(inputs, self.gamma, self.beta, axis=axis, epsilon=self.epsilon)
        return y

    call = forward

    def get_weights(self):
        return [self.gamma.detach().cpu().numpy(), self.beta.detach().cpu().numpy()]

    def set_weights(self, weights):
        gamma, beta = weights
        with torch.no_grad():
            self.gamma.copy_(torch.as_tensor(gamma, dtype=torch.float32).reshape(self.gamma.shape))
            self.beta.copy_(torch.as_tensor(beta, dtype=torch.float32).reshape(self.beta.shape))

    @property
    def variables(self):
        return [self.gamma, self.beta]

    def get_config(self):
        return {"axis": self.axis, "epsilon": self.epsilon}


class InstanceNormalization(torch.nn.Module):
    """Same contract as the reference layer (nv_norm_ops.py:123-184): `axis` is the channel
    axis and must be 1 (channel-first, "NC...") or -1 (channels-last, "N...C"); weights are
    float32 [C] whatever the activation dtype; output is `y` only.
    """

    def __init__(self, axis: int = -1, epsilon: float = 1e-3, **kwargs):
        super().__init__()
        unsupported = {k: v for k, v in kwargs.items()
                       if k in ("center", "scale") and v is not True}
        if unsupported:
            raise ValueError(f"the fused op always centers and scales; got {unsupported}")
        self.axis = axis
        self.epsilon = float(epsilon)
        self.gamma = None
        self.beta = None
        self.built = False

    def build(self, input_shape, device=None):
        c = int(input_shape[self.axis])
        self.gamma = torch.nn.Parameter(torch.ones(c, dtype=torch.float32, device=device))
        self.beta = torch.nn.Parameter(torch.zeros(c, dtype=torch.float32, device=device))
        self.built = True

    def forward(self, inputs):
        if not self.built:
            self.build(tuple(inputs.shape), device=inputs.device)
        axis = self.axis
        if axis == 1:
            data_format = "NC..."
        elif axis == -1:
            data_format = "N...C"
        else:
            raise ValueError("We only support integer axis of 1 or -1 corresponds to channel "
                             "first or channel last layout.")
        y, _, _ = fused_instance_norm(inputs, self.gamma, self.beta, data_format=data_format,
                                      epsilon=self.epsilon)
        return y

    call = forward

    def get_weights(self):
        return [self.gamma.detach().cpu().numpy(), self.beta.detach().cpu().numpy()]

    def set_weights(self, weights):
        gamma, beta = weights
        with torch.no_grad():
            self.gamma.copy_(torch.as_tensor(gamma, dtype=torch.float32).reshape(self.gamma.shape))
            self.beta.copy_(torch.as_tensor(beta, dtype=torch.float32).reshape(self.beta.shape))

    @property
    def variables(self):
        return [self.gamma, self.beta]

    def get_config(self):
        return {"axis": self.axis, "epsilon": self.epsilon}
