"""User-facing configuration types (same names, fields and defaults as the reference's
``float8_experimental/config.py``, so configs written for it construct unchanged)."""
import enum
from dataclasses import dataclass, field


class ScalingType(enum.Enum):
    """How the scale of one tensor is obtained (reference config.py:12-21)."""

    DELAYED = "delayed"  # from the amax history of earlier iterations
    DYNAMIC = "dynamic"  # from the tensor itself, every time

    def short_str(self) -> str:
        return {ScalingType.DELAYED: "del", ScalingType.DYNAMIC: "dyn"}[self]


@dataclass(frozen=True)
class CastConfig:
    """Casting recipe of a single tensor (reference config.py:24-30)."""

    scaling_type: ScalingType = ScalingType.DYNAMIC


@dataclass(frozen=True)
class DelayedScalingConfig:
    """Delayed-scaling recipe shared by every tensor and layer (reference config.py:33-54)."""

    history_len: int = 16  # length of each amax history buffer
    scale_fn_name: str = "max"  # reduction of the history to one amax

    def __post_init__(self):
        if self.scale_fn_name != "max":
            raise AssertionError(f"{self.scale_fn_name} is not implemented yet. Only max is supported for now.")


@dataclass(frozen=True)
class Float8GemmConfig:
    """Per-GEMM knobs (reference config.py:57-65).

    ``use_fast_accum`` is accepted for compatibility; the gfx950 matrix cores have a
    single fp32 accumulation mode, so it changes nothing here.
    """

    use_fast_accum: bool = False


@dataclass(frozen=True)
class Float8LinearConfig:
    """Everything ``convert_to_float8_training`` needs (reference config.py:68-123)."""

    # one recipe per tensor taking part in the three GEMMs
    cast_config_input: CastConfig = CastConfig()
    cast_config_weight: CastConfig = CastConfig()
    cast_config_grad_output: CastConfig = CastConfig()

    # one per GEMM: output = x W^T, grad_input = dY W, grad_weight = dY^T x
    gemm_config_output: Float8GemmConfig = Float8GemmConfig(use_fast_accum=True)
    gemm_config_grad_input: Float8GemmConfig = Float8GemmConfig()
    gemm_config_grad_weight: Float8GemmConfig = Float8GemmConfig()

    # initialise amax/history/scale from the data seen in the first iteration
    enable_amax_init: bool = True
    # run the synced/initialised bookkeeping around forward
    enable_pre_and_post_forward: bool = True
    # FSDP2 float8 all-gather of the weight: on one GPU nothing is gathered; the flag marks the weights whose
    # scales precompute_float8_dynamic_scale_for_fsdp computes ahead of the forward pass
    enable_fsdp_float8_all_gather: bool = False
    # zero-pad the reduction dimension to a multiple of 16 before the GEMM; the kernel
    # here handles ragged shapes itself, so the flag is accepted and has no effect on results
    pad_inner_dim: bool = False
    # compute the three matmuls in fp32 from dequantised operands instead of on the matrix cores
    emulate: bool = False

    delayed_scaling_config: DelayedScalingConfig = DelayedScalingConfig()


# The reference can switch to the "fnuz" fp8 flavours of older AMD GPUs through this module
# global.  gfx950 implements the OCP formats natively, so only False is supported.
use_fnuz_dtype = False
