"""atex_amd: MI355X-native implementation of NVIDIA/atex's nv_norms hot path."""
from . import nv_norms  # noqa: F401
