"""atex_amd.nv_norms: fused LayerNorm / InstanceNorm for MI355X behind the public names of
the reference package (atex/nv_norms/__init__.py:6-13)."""
from ._capi import AtexnError, InvalidArgumentError  # noqa: F401
from .layers import InstanceNormalization  # noqa: F401
from .layers import LayerNormalization  # noqa: F401
from .layers import _instance_norm_grad  # noqa: F401
from .layers import _layer_norm_grad  # noqa: F401
from .layers import fused_instance_norm, fused_layer_norm  # noqa: F401
from .ops import fused_instance_norm_grad_op  # noqa: F401
from .ops import fused_instance_norm_op  # noqa: F401
from .ops import fused_layer_norm_grad_op  # noqa: F401
from .ops import fused_layer_norm_op  # noqa: F401
