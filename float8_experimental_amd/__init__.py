"""MI355X-native Float8Linear hot path behind float8_experimental's Python API.

Same top-level names as the reference's ``float8_experimental/__init__.py``; the
arithmetic underneath runs as hand-written gfx950 kernels loaded through a C ABI
(``libf8mi.so``, declared in ``include/f8mi.h``).
"""
from .config import CastConfig, DelayedScalingConfig, Float8GemmConfig, Float8LinearConfig, ScalingType
from .float8_linear import Float8Linear
from .float8_linear_utils import (
    convert_to_float8_training,
    get_float8_layers,
    linear_requires_sync,
    sync_float8_amax_and_scale_history,
)
from .float8_tensor import Float8Tensor, GemmInputRole, LinearMMConfig, ScaledMMConfig
from .fsdp_utils import precompute_float8_dynamic_scale_for_fsdp

from torch.serialization import add_safe_globals

# lets torch.load(..., weights_only=True) rebuild Float8Tensors
add_safe_globals([Float8Tensor, ScaledMMConfig, GemmInputRole, LinearMMConfig])

__all__ = [
    "DelayedScalingConfig",
    "ScalingType",
    "Float8GemmConfig",
    "Float8LinearConfig",
    "CastConfig",
    "convert_to_float8_training",
    "linear_requires_sync",
    "sync_float8_amax_and_scale_history",
    "precompute_float8_dynamic_scale_for_fsdp",
]
