"""Operator table of ``Float8Tensor`` (mirror of the reference's ``float8_ops.py``).

``Float8Tensor.__torch_dispatch__`` looks every aten op up in ``FLOAT8_OPS_TABLE``;
anything not listed raises ``NotImplementedError``.  The collective handlers of the
reference (``all_gather_into_tensor`` / ``wait_tensor``) belong to its multi-GPU
flows and are not part of this build.
"""
from typing import Any, Dict

import torch
from torch.utils._pytree import tree_map

from . import float8_aten_api  # noqa: F401  (registers torch.ops.aten.mm_float8_emulated)
from .float8_python_api import addmm_float8_unwrapped
from .float8_tensor import choose_scaled_mm_config, Float8Tensor
from .float8_utils import pad_tensor_for_matmul

aten = torch.ops.aten
FLOAT8_OPS_TABLE: Dict[Any, Any] = {}


def implements(aten_ops):
    """Decorator: register ``func`` as the handler of each op in ``aten_ops``."""

    def register(func):
        for op in aten_ops:
            FLOAT8_OPS_TABLE[op] = func
        return func

    return register


def _like(src: Float8Tensor, data: torch.Tensor, orig_dtype=None) -> Float8Tensor:
    """A Float8Tensor over ``data`` with the scale and GEMM bookkeeping of ``src``."""
    return Float8Tensor(data, src._scale, src._orig_dtype if orig_dtype is None else orig_dtype,
                        src._linear_mm_config, src._gemm_input_role)


def _same_family(a: Float8Tensor, b: Float8Tensor, what: str, scale_by_identity: bool) -> None:
    assert a._orig_dtype == b._orig_dtype, f"Expecting {what} to be of the same dtype"
    if scale_by_identity:
        assert a._scale is b._scale, f"Expecting {what} to have the same scale as a result of a split"
        assert a._linear_mm_config is b._linear_mm_config, f"Expecting {what} to have the same mm config as a result of a split"
    else:
        assert a._scale == b._scale, f"Expecting {what} to have the same scale"
        assert a._linear_mm_config == b._linear_mm_config, f"Expecting {what} to have the same mm config"
    assert a._data.dtype == b._data.dtype, f"Expecting {what} to be of the same float8 dtype"
    assert a._gemm_input_role is b._gemm_input_role, f"Expecting {what} to have the same gemm_input_role"


# ---- ops that only re-view or refill the payload (reference float8_ops.py:33-54)
@implements([aten.view.default, aten._unsafe_view.default, aten.t.default, aten.as_strided.default,
             aten.clone.default, aten.detach.default, aten.slice.Tensor, aten.transpose.int, aten.fill_.Scalar])
def float8_desugar_op(aten_op, args, kwargs=None):
    return _like(args[0], aten_op(args[0]._data, *args[1:], **(kwargs or {})))


@implements([aten.split.Tensor])
def float8_split(aten_op, args, kwargs=None):
    """Pieces share the parent's scale object (reference :57-71)."""
    return [_like(args[0], piece) for piece in aten_op(args[0]._data, *args[1:], **(kwargs or {}))]


@implements([aten.cat.default])
def float8_cat(aten_op, args, kwargs=None):
    """Concatenates pieces of one split, through a byte view (reference :75-108)."""
    chunks = args[0]
    first = chunks[0]
    payloads = []
    for chunk in chunks:
        assert isinstance(chunk, Float8Tensor), "Expecting all chunks to be of type Float8Tensor"
        _same_family(first, chunk, "all chunks", scale_by_identity=True)
        payloads.append(chunk._data.view(torch.uint8))
    joined = aten_op(payloads, *args[1:], **(kwargs or {})).view(first._data.dtype)
    return _like(first, joined)


@implements([aten.sum.dim_IntList])
def float8_cast_up_op(aten_op, args, kwargs=None):
    """Runs the op on the dequantised tensor; needed by addmm's bias gradient (reference :111-128)."""
    up = lambda x: x.to_original_precision() if isinstance(x, Float8Tensor) else x
    return aten_op(*tree_map(up, args), **tree_map(up, kwargs or {}))


def preprocess_addmm(a: Float8Tensor, b: Float8Tensor):
    """Operands of ``a @ b`` for ``addmm_float8_unwrapped`` (reference :131-155).  ``pad_inner_dim`` zero-pads the
    reduction to a multiple of 16 exactly like the reference; zeros do not change the product and the kernel needs
    no padding.  The reference goes on to copy the payloads into the one layout ``torch._scaled_mm`` takes -- ``a``
    row-major, ``b`` column-major (:150-153); here they are handed on as they lie: the kernel behind
    ``addmm_float8_unwrapped`` reads a row-major ``b`` (and a column-major ``a``) transposed, and makes that copy
    itself only for the small or ragged products where it cannot."""
    a_data, b_data = a._data, b._data
    cfg = choose_scaled_mm_config(a._gemm_input_role, a._linear_mm_config, b._gemm_input_role, b._linear_mm_config)
    if cfg.pad_inner_dim:
        assert a_data.size(1) == b_data.size(0), f"Inner dims must match for mm, got {a_data.size(1)} and {b_data.size(0)}"
        a_data = pad_tensor_for_matmul(a_data, dims=1)
        b_data = pad_tensor_for_matmul(b_data, dims=0)
    return a_data, a._scale, b_data, b._scale


def _mm_impl(a: Float8Tensor, b: Float8Tensor, bias):
    assert isinstance(a, Float8Tensor) and isinstance(b, Float8Tensor), (
        "Expecting  both Float8Tensor for mm inputs but found {} and {}".format(type(a), type(b)))
    a_data, a_scale, b_data, b_scale = preprocess_addmm(a, b)
    cfg = choose_scaled_mm_config(a._gemm_input_role, a._linear_mm_config, b._gemm_input_role, b._linear_mm_config)
    output_dtype = a._orig_dtype
    if cfg.emulate:
        out = torch.ops.aten.mm_float8_emulated(a._data, a._scale, b._data, b._scale, output_dtype)
        return out if bias is None else out + bias
    return addmm_float8_unwrapped(a_data, a_scale, b_data, b_scale, output_dtype, output_scale=None, bias=bias,
                                  use_fast_accum=cfg.use_fast_accum)


@implements([aten.mm.default, aten.matmul.default])
def float8_mm(aten_op, args, kwargs=None):
    """fp8 x fp8 matmul with the settings the operands' roles select (reference :158-190)."""
    return _mm_impl(args[0], args[1], None)


@implements([aten.addmm.default])
def float8_addmm(aten_op, args, kwargs=None):
    """``bias + a @ b`` (reference :193-227)."""
    assert isinstance(args[0], torch.Tensor) and isinstance(args[1], Float8Tensor) and isinstance(args[2], Float8Tensor)
    assert args[0].dtype == args[1]._orig_dtype, "bias dtype must match output dtype"
    return _mm_impl(args[1], args[2], args[0])


@implements([aten.is_same_size.default])
def float8_is_same_size(aten_op, args, kwargs=None):
    return args[0].shape == args[1].shape


@implements([aten._to_copy.default])
def autocast_to_copy(aten_op, args, kwargs=None):
    """Under autocast a Float8Tensor is "converted" by relabelling what it presents as (reference :235-255)."""
    kwargs = kwargs or {}
    assert isinstance(args[0], Float8Tensor)
    assert len(kwargs) == 1 and "dtype" in kwargs, "Only support dtype kwarg for autocast"
    assert kwargs["dtype"] in {torch.float16, torch.bfloat16}, (
        "Only support floating point conversion for autocast w/ Float8Tensor")
    return _like(args[0], args[0]._data, orig_dtype=kwargs["dtype"])


@implements([aten.index_put_.default])
def index_put_fp8(aten_op, args, kwargs=None):
    """In-place indexed write between Float8Tensors of one scale (reference :301-320)."""
    dst, values = args[0], args[2]
    assert isinstance(dst, Float8Tensor) and isinstance(values, Float8Tensor)
    assert dst._scale == values._scale
    assert dst.dtype == values.dtype
    assert dst._orig_dtype == values._orig_dtype
    return _like(dst, aten_op(dst._data, args[1], values._data, *args[3:], **(kwargs or {})))


@implements([aten.copy_.default])
def copy_fp8(aten_op, args, kwargs=None):
    """hp <- fp8 dequantises; fp8 <- fp8 needs identical metadata; fp8 <- hp is refused (reference :323-363)."""
    dst, src = args[0], args[1]
    kwargs = kwargs or {}
    if isinstance(src, Float8Tensor) and not isinstance(dst, Float8Tensor):
        return aten_op(dst, src.to_original_precision(), *args[2:], **kwargs)
    if isinstance(src, Float8Tensor) and isinstance(dst, Float8Tensor):
        _same_family(dst, src, "both Float8Tensors", scale_by_identity=False)
        return _like(dst, aten_op(dst._data, src._data, *args[2:], **kwargs))
    raise RuntimeError("Unsupported semantics for copy_ in Float8Tensor")
