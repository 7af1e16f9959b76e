"""``Float8Tensor``: fp8 payload + scale + GEMM bookkeeping as one tensor
(mirror of the reference's ``float8_tensor.py``; DTensor branches are out of scope).
"""
import enum
from collections import namedtuple
from typing import Dict, Optional

import torch

from . import _native
from .float8_utils import e4m3_dtype

# Per-GEMM settings (reference float8_tensor.py:55-59).  ``use_fast_accum`` and
# ``pad_inner_dim`` are carried for compatibility and do not change results here.
ScaledMMConfig = namedtuple(
    "ScaledMMConfig",
    ["emulate", "use_fast_accum", "fp8_output", "pad_inner_dim"],
    defaults=[False, False, False, False],
)

# The three GEMMs of a linear layer (reference float8_tensor.py:66-74).
LinearMMConfig = namedtuple(
    "LinearMMConfig",
    ["output", "grad_input", "grad_weight"],
    defaults=[
        ScaledMMConfig(False, True, False, False),
        ScaledMMConfig(False, False, False, False),
        ScaledMMConfig(False, False, False, False),
    ],
)


class GemmInputRole(enum.Enum):
    """Which of the three tensors of a linear layer a Float8Tensor is (reference :77-87)."""

    INPUT = "input"
    WEIGHT = "weight"
    GRAD_OUTPUT = "grad_output"


_GEMM_OF_ROLES = {
    (GemmInputRole.INPUT, GemmInputRole.WEIGHT): "output",
    (GemmInputRole.GRAD_OUTPUT, GemmInputRole.WEIGHT): "grad_input",
    (GemmInputRole.GRAD_OUTPUT, GemmInputRole.INPUT): "grad_weight",
}


def choose_scaled_mm_config(a_role, a_linear_mm_config, b_role, b_linear_mm_config) -> ScaledMMConfig:
    """Settings of the GEMM ``a @ b`` from the operands' roles (reference :91-113)."""
    which = _GEMM_OF_ROLES.get((a_role, b_role))
    if which is None:
        raise AssertionError(f"unexpected a_role {a_role} and b_role {b_role}")
    mine, theirs = getattr(a_linear_mm_config, which), getattr(b_linear_mm_config, which)
    assert mine == theirs, f"linear_mm_config.{which} mismatch: {mine} vs {theirs}"
    return mine


def tensor_already_casted_to_fp8(tensor: torch.Tensor) -> bool:
    """True for a Float8Tensor (reference :116-128; the DTensor / async-collective wrappers
    looked through there belong to multi-GPU flows)."""
    return isinstance(tensor, Float8Tensor)


def _product_dtype(hp: torch.Tensor, scale: torch.Tensor) -> torch.dtype:
    """dtype torch's promotion gives ``hp * scale``: a 0-dim fp32 scale leaves hp's dtype,
    a scale with a dimension (the [1]-shaped delayed-scaling buffers) promotes to fp32."""
    if scale.dim() == 0 and hp.dim() > 0:
        return hp.dtype
    return torch.promote_types(hp.dtype, scale.dtype)


@torch._dynamo.allow_in_graph
class _ToFloat8ConstrFunc(torch.autograd.Function):
    """High precision -> Float8Tensor; the gradient passes through unchanged (reference :131-195).
    The cast is the custom op ``f8mi::cast``: one opaque node when ``torch.compile`` traces this function."""

    @staticmethod
    def forward(ctx, tensor, scale, float8_dtype=e4m3_dtype, linear_mm_config=None,
                gemm_input_role=GemmInputRole.INPUT, amax_buffer=None):
        _native._require_gpu(tensor, "tensor")
        plain = (torch.Tensor, torch.nn.Parameter)
        if (amax_buffer is not None and not torch.compiler.is_compiling() and type(tensor) in plain
                and type(amax_buffer) in plain and amax_buffer.dtype == torch.float32 and amax_buffer.numel() == 1):
            # eager mode, delayed scaling: the kernel writes max|tensor| into the module's buffer itself (no
            # temporary, no copy launch)
            bits, _ = _native.cast(tensor, scale, float8_dtype, product_dtype=_product_dtype(tensor, scale), amax_out=amax_buffer)
        else:
            # one opaque node for torch.compile; functional, so the amax comes back and is copied into the buffer
            bits, amax = torch.ops.f8mi.cast(tensor, scale, float8_dtype, _product_dtype(tensor, scale), amax_buffer is not None)
            if amax_buffer is not None:
                amax_buffer.copy_(amax.reshape(amax_buffer.shape))
        return Float8Tensor(bits, scale, tensor.dtype, linear_mm_config=linear_mm_config,
                            gemm_input_role=gemm_input_role)

    @staticmethod
    def backward(ctx, g):
        return g, None, None, None, None, None, None


@torch._dynamo.allow_in_graph
class _FromFloat8ConstrFunc(torch.autograd.Function):
    """Float8Tensor -> high precision; the gradient passes through unchanged (reference :198-212)."""

    @staticmethod
    def forward(ctx, tensor):
        return tensor._data.to(tensor._orig_dtype) / tensor._scale

    @staticmethod
    def backward(ctx, g):
        return g, None, None


def hp_tensor_and_scale_to_float8(hp_tensor: torch.Tensor, s: torch.Tensor, float8_dtype=e4m3_dtype,
                                  linear_mm_config: Optional[LinearMMConfig] = None,
                                  gemm_input_role: Optional[GemmInputRole] = GemmInputRole.INPUT):
    """fp8(clamp(hp_tensor * s)) wrapped as a Float8Tensor, differentiable as identity (reference :215-240)."""
    return _ToFloat8ConstrFunc.apply(hp_tensor, s, float8_dtype, linear_mm_config, gemm_input_role)


class Float8Tensor(torch.Tensor):
    """Wrapper subclass bundling (reference float8_tensor.py:243-363):

    * ``_data``   the fp8 payload (``float8_e4m3fn`` or ``float8_e5m2``),
    * ``_scale``  one fp32 element; high precision * scale = fp8 range,
    * ``_orig_dtype``  what the tensor presents itself as,
    * ``_linear_mm_config`` / ``_gemm_input_role``  which GEMM settings apply when it is multiplied.

    Operators reach ``FLOAT8_OPS_TABLE`` of ``float8_ops`` through ``__torch_dispatch__``.
    """

    __slots__ = ["_data", "_scale", "_orig_dtype", "_linear_mm_config", "_gemm_input_role"]

    def __new__(cls, data: torch.Tensor, scale: torch.Tensor, orig_dtype: torch.dtype,
                linear_mm_config: Optional[LinearMMConfig], gemm_input_role: Optional[GemmInputRole] = GemmInputRole.INPUT):
        assert scale.numel() == 1, "Scale should contain a single value, but got: {} elements".format(scale.numel())
        self = torch.Tensor._make_wrapper_subclass(
            cls, data.size(), strides=data.stride(), storage_offset=data.storage_offset(), dtype=orig_dtype,
            layout=data.layout, requires_grad=data.requires_grad, device=data.device,
        )
        self._data = data
        self._scale = scale
        self._orig_dtype = orig_dtype
        self._linear_mm_config = linear_mm_config if linear_mm_config is not None else LinearMMConfig()
        self._gemm_input_role = gemm_input_role
        return self

    def __repr__(self):
        return (f"Float8Tensor(dtype={self._data.dtype}, scale={self._scale}, "
                f"linear_mm_config={self._linear_mm_config}\ngemm_input_role={self._gemm_input_role}\n"
                f"as_orig_prec={self.to_original_precision()}")

    def __tensor_flatten__(self):
        meta = {"_orig_dtype": self._orig_dtype, "_linear_mm_config": self._linear_mm_config,
                "_gemm_input_role": self._gemm_input_role}
        return ["_data", "_scale"], meta

    @staticmethod
    def __tensor_unflatten__(inner_tensors: Dict, metadata, outer_size, outer_stride):
        assert len(inner_tensors) == 2
        return Float8Tensor(inner_tensors["_data"], inner_tensors["_scale"], metadata["_orig_dtype"],
                            metadata["_linear_mm_config"], metadata["_gemm_input_role"])

    def to_original_precision(self):
        return _FromFloat8ConstrFunc.apply(self)

    @classmethod
    def __torch_dispatch__(cls, func, types, args, kwargs=None):
        from .float8_ops import FLOAT8_OPS_TABLE  # late: float8_ops imports this module

        # mixed subclasses are left to the other subclass's handler
        def known(t):
            return (issubclass(cls, t) or issubclass(torch._subclasses.fake_tensor.FakeTensor, t)
                    or issubclass(torch._subclasses.functional_tensor.FunctionalTensor, t))

        if not all(known(t) for t in types):
            return NotImplemented
        handler = FLOAT8_OPS_TABLE.get(func)
        if handler is None:
            raise NotImplementedError(f"attempting to run {func}, this is not supported")
        return handler(func, args, kwargs if kwargs is not None else {})

    # results of torch functions are not re-wrapped as Float8Tensor
    __torch_function__ = torch._C._disabled_torch_function_impl
