"""nv_norms for TensorFlow-ROCm: the reference package's public names
(atex/nv_norms/__init__.py:6-13) on top of `_fused_nv_norm_ops.so`, the op library built from
this directory (op registrations + OpKernels calling libatex_norms_hip.so).

Needs TensorFlow (ROCm build) at import time.  `tensorflow_addons` is imported only when an
`InstanceNormalization` layer is created, so LayerNormalization and the four raw ops work
without it (the reference imports it unconditionally, python/ops/nv_norm_ops.py:12).
"""
from .ops import (InstanceNormalization, LayerNormalization, _instance_norm_grad, _layer_norm_grad,
                  fused_instance_norm_grad_op, fused_instance_norm_op, fused_layer_norm_grad_op,
                  fused_layer_norm_op)

__all__ = [
    "LayerNormalization", "InstanceNormalization", "fused_layer_norm_op", "fused_layer_norm_grad_op",
    "fused_instance_norm_op", "fused_instance_norm_grad_op", "_layer_norm_grad", "_instance_norm_grad",
]
