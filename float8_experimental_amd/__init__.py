"""MI355X-native Float8Linear hot path behind float8_experimental's Python API.

Same top-level names as the reference's ``float8_experimental/__init__.py``; the
arithmetic underneath runs as hand-written gfx950 kernels loaded through a C ABI
(``libf8mi.so``, declared in ``include/f8mi.h``).
"""
import torch.serialization as _serialization

# configuration: what a user writes down before converting a model
from .config import ScalingType  # dynamic or delayed, per tensor
from .config import CastConfig  # the recipe of one of input / weight / grad_output
from .config import DelayedScalingConfig  # history length and reduction, shared by all layers
from .config import Float8GemmConfig  # per-GEMM knobs (accepted, one accumulation mode here)
from .config import Float8LinearConfig  # all of the above for one conversion

# the module, the model-level helpers around it, and the tensor type the op-by-op route passes along
from .float8_linear import Float8Linear
from .float8_linear_utils import convert_to_float8_training  # swap nn.Linear -> Float8Linear
from .float8_linear_utils import get_float8_layers
from .float8_linear_utils import linear_requires_sync  # does a config use delayed scaling anywhere?
from .float8_linear_utils import sync_float8_amax_and_scale_history  # once per step, before forward
from .float8_tensor import Float8Tensor, GemmInputRole, LinearMMConfig, ScaledMMConfig
from .fsdp_utils import precompute_float8_dynamic_scale_for_fsdp  # all weight scales in one pass

# checkpoints holding Float8Tensors load with torch.load(..., weights_only=True)
_serialization.add_safe_globals([Float8Tensor, GemmInputRole, LinearMMConfig, ScaledMMConfig])

# the reference's public names, in the order a training script meets them
__all__ = ["ScalingType", "CastConfig", "DelayedScalingConfig", "Float8GemmConfig", "Float8LinearConfig",
           "convert_to_float8_training", "linear_requires_sync", "sync_float8_amax_and_scale_history",
           "precompute_float8_dynamic_scale_for_fsdp"]
