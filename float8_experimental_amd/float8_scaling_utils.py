"""High precision -> float8 with dynamic or delayed scaling
(mirror of the reference's ``float8_scaling_utils.py``).
"""
from typing import Optional

import torch

from . import _native
from .float8_tensor import (
    _ToFloat8ConstrFunc,
    Float8Tensor,
    GemmInputRole,
    hp_tensor_and_scale_to_float8,
    LinearMMConfig,
    tensor_already_casted_to_fp8,
)
from .float8_utils import _no_multi_rank, e4m3_dtype, e5m2_dtype, tensor_to_scale


def hp_tensor_to_float8_dynamic(hp_tensor: torch.Tensor, float8_dtype: torch.dtype, linear_mm_config: LinearMMConfig,
                                reduce_amax: bool = False,
                                gemm_input_role: GemmInputRole = GemmInputRole.INPUT) -> Float8Tensor:
    """Scale from the tensor's own amax, then cast (reference float8_scaling_utils.py:33-62)."""
    if tensor_already_casted_to_fp8(hp_tensor):
        return hp_tensor
    scale = tensor_to_scale(hp_tensor, float8_dtype, reduce_amax)
    return hp_tensor_and_scale_to_float8(hp_tensor, scale, float8_dtype, linear_mm_config, gemm_input_role)


def hp_tensor_to_float8_delayed(hp_tensor: torch.Tensor, s: torch.Tensor, float8_dtype: torch.dtype,
                                amax_buffer: torch.Tensor, linear_mm_config: Optional[LinearMMConfig] = None,
                                gemm_input_role: Optional[GemmInputRole] = GemmInputRole.INPUT) -> Float8Tensor:
    """Cast with the given (older) scale and record this tensor's amax in ``amax_buffer``
    (reference float8_scaling_utils.py:65-96).  The amax pass is folded into the cast kernel
    here (one read of the tensor instead of two); the values are the same."""
    return _ToFloat8ConstrFunc.apply(hp_tensor, s, float8_dtype, linear_mm_config, gemm_input_role, amax_buffer)


def _maybe_initialize_amaxes_scales_for_float8_cast(x, cur_amax, amax_history, scale, scale_fn_name, float8_dtype,
                                                    is_initialized, reduce_amax):
    """First iteration only: amax <- max|x|, history[0] <- amax, scale <- f(max(history))
    (reference float8_scaling_utils.py:99-125)."""
    if is_initialized:
        return
    if scale_fn_name != "max":
        raise NotImplementedError()
    _no_multi_rank(reduce_amax)
    with torch.no_grad():
        _native.amax_scale(x, float8_dtype, want_scale=False, amax_out=cur_amax)
        _native.delayed_init(cur_amax, amax_history, scale, float8_dtype, x.dtype == torch.float16)


@torch._dynamo.allow_in_graph
class NoopFwToFloat8E5M2BwDelayed(torch.autograd.Function):
    """Identity in forward; casts the gradient to e5m2 with delayed scaling in backward
    (reference float8_scaling_utils.py:128-185)."""

    @staticmethod
    def forward(ctx, tensor, fp8_amax_grad_output, fp8_amax_history_grad_output, fp8_scale_grad_output,
                scale_fn_name, is_amax_initialized, linear_mm_config: LinearMMConfig):
        ctx.save_for_backward(fp8_amax_grad_output, fp8_amax_history_grad_output, fp8_scale_grad_output)
        ctx.scale_fn_name = scale_fn_name
        ctx.is_amax_initialized = is_amax_initialized
        ctx.linear_mm_config = linear_mm_config
        return tensor

    @staticmethod
    def backward(ctx, go):
        amax, history, scale = ctx.saved_tensors
        _maybe_initialize_amaxes_scales_for_float8_cast(go, amax, history, scale, ctx.scale_fn_name, e5m2_dtype,
                                                        ctx.is_amax_initialized, reduce_amax=True)
        res = hp_tensor_to_float8_delayed(go, scale, e5m2_dtype, amax, ctx.linear_mm_config,
                                          GemmInputRole.GRAD_OUTPUT)
        return res, None, None, None, None, None, None


@torch._dynamo.allow_in_graph
class NoopFwToFloat8E5M2BwDynamic(torch.autograd.Function):
    """Identity in forward; casts the gradient to e5m2 with dynamic scaling in backward
    (reference float8_scaling_utils.py:188-216)."""

    @staticmethod
    def forward(ctx, tensor, linear_mm_config: LinearMMConfig):
        ctx.linear_mm_config = linear_mm_config
        return tensor

    @staticmethod
    def backward(ctx, gradY):
        if tensor_already_casted_to_fp8(gradY):
            return gradY, None
        scale = tensor_to_scale(gradY, e5m2_dtype)
        return hp_tensor_and_scale_to_float8(gradY, scale, e5m2_dtype, ctx.linear_mm_config,
                                             GemmInputRole.GRAD_OUTPUT), None
