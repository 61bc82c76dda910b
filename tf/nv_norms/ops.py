"""Python side of the fused normalisation ops under TensorFlow: loads the op library, registers
the gradients, and provides the two Keras layers.  Same names, arguments and behaviour as the
reference's python/ops/nv_norm_ops.py (cited per item below)."""
import os

import tensorflow as tf
from tensorflow.python.framework import load_library, ops as tf_ops

_OP_LIBRARY = "_fused_nv_norm_ops.so"


def _find_op_library():
    """ATEXN_TF_OP_LIBRARY if set, else the library beside this package or one level up (where
    the CMake install rule puts it; the reference keeps its library at the site-packages root,
    nv_norm_ops.py:19-21)."""
    env = os.environ.get("ATEXN_TF_OP_LIBRARY")
    here = os.path.dirname(os.path.abspath(__file__))
    for cand in ([env] if env else []) + [os.path.join(here, _OP_LIBRARY), os.path.join(here, "..", _OP_LIBRARY)]:
        if os.path.exists(cand):
            return cand
    raise ImportError(f"{_OP_LIBRARY} not found (build tf/ with CMake, or set ATEXN_TF_OP_LIBRARY)")


_lib = load_library.load_op_library(_find_op_library())
fused_layer_norm_op = _lib.fused_layer_norm
fused_layer_norm_grad_op = _lib.fused_layer_norm_grad
fused_instance_norm_op = _lib.fused_instance_norm
fused_instance_norm_grad_op = _lib.fused_instance_norm_grad


def _saved_state(op):
    """(x, gamma, saved mean, saved inverse std) of a forward op."""
    return op.inputs[0], op.inputs[1], op.outputs[1], op.outputs[2]


@tf_ops.RegisterGradient("FusedLayerNorm")
def _layer_norm_grad(op, *grad):
    """Gradient of FusedLayerNorm with respect to x, scale, offset (nv_norm_ops.py:48-67): the
    grad op gets the incoming gradient of y, the forward inputs and saved statistics, and the
    forward op's `axis`; epsilon is not needed."""
    x, gamma, mean, inv_std = _saved_state(op)
    return list(fused_layer_norm_grad_op(grad[0], x, gamma, mean, inv_std, axis=op.get_attr("axis")))


@tf_ops.RegisterGradient("FusedInstanceNorm")
def _instance_norm_grad(op, *grad):
    """Gradient of FusedInstanceNorm (nv_norm_ops.py:27-46), with the forward op's `data_format`."""
    x, gamma, mean, inv_std = _saved_state(op)
    return list(fused_instance_norm_grad_op(grad[0], x, gamma, mean, inv_std,
                                            data_format=op.get_attr("data_format")))


class _FusedNormLayer(tf.keras.layers.Layer):
    """A Keras layer whose weights live in a private stock layer (`self._holder`), used only to
    create, name and (de)serialise gamma / beta the way the stock layer would; the forward pass
    is the fused op.  Weight access is delegated (nv_norm_ops.py:101-121, 166-184)."""

    _holder_key = "holder"

    def __init__(self, holder):
        super().__init__()
        self._holder = holder

    def build(self, input_shape):
        self._holder.build(input_shape=input_shape)
        self.built = True

    def get_weights(self):
        return self._holder.get_weights()

    def set_weights(self, weights):
        self._holder.set_weights(weights)

    @property
    def variables(self):
        return self._holder.weights

    def get_config(self):
        config = dict(super().get_config())
        config[self._holder_key] = self._holder
        return config


class LayerNormalization(_FusedNormLayer):
    """Arguments of tf.keras.layers.LayerNormalization, forwarded to the private stock layer; the
    wrapper's own name and dtype stay the defaults (nv_norm_ops.py:77-79).  `axis` must cover a
    contiguous run of dimensions ending at the last one.  Returns y only."""

    _holder_key = "layer_norm"

    def __init__(self, **kwargs):
        super().__init__(tf.keras.layers.LayerNormalization(**kwargs))

    @property
    def layer_norm(self):
        return self._holder

    def call(self, inputs):
        axis = self._holder.axis  # negatives already wrapped by the stock layer's build()
        axis = [axis] if isinstance(axis, int) else list(axis)
        if axis != sorted(set(axis)):
            raise ValueError("We only support sorted and unique axis to make sure the weights have the "
                             "same data layout with the keras layers.")
        y, _, _ = fused_layer_norm_op(inputs, self._holder.gamma, self._holder.beta, axis=axis,
                                      epsilon=self._holder.epsilon)
        return y


class InstanceNormalization(_FusedNormLayer):
    """Arguments of tfa.layers.InstanceNormalization; `axis` is 1 (channel first) or -1 (channels
    last).  The op wants float32 gamma / beta, so the private layer is created under the
    float32 policy even when the global policy is a mixed one (nv_norm_ops.py:130-143)."""

    _holder_key = "instance_norm"

    def __init__(self, axis, **kwargs):
        import tensorflow_addons as tfa  # only needed here

        policy = tf.keras.mixed_precision.global_policy()
        mixed = policy is not None and policy.compute_dtype != policy.variable_dtype
        if mixed:
            tf.keras.mixed_precision.set_global_policy("float32")
        try:
            holder = tfa.layers.InstanceNormalization(axis=axis, **kwargs)
        finally:
            if mixed:
                tf.keras.mixed_precision.set_global_policy(policy)
        super().__init__(holder)

    @property
    def instance_norm(self):
        return self._holder

    def call(self, inputs):
        axis = self._holder.axis
        if axis not in (1, -1):
            raise ValueError("We only support integer axis of 1 or -1 corresponds to channel first or "
                             "channel last layout.")
        y, _, _ = fused_instance_norm_op(inputs, self._holder.weights[0], self._holder.weights[1],
                                         data_format="NC..." if axis == 1 else "N...C",
                                         epsilon=self._holder.epsilon)
        return y
