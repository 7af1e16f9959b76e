"""Numeric primitives of the float8 path (mirror of the reference's ``float8_utils.py``).

amax, scale and the saturated cast run as hand-written gfx950 kernels behind the
C ABI (``_native``); tensors must live on the GPU.
"""
from typing import Iterable, Literal, Tuple, Union

import torch

from . import _custom_ops  # noqa: F401  (registers torch.ops.f8mi.*)
from . import _native
from . import config as _config

EPS = 1e-12  # floor of amax when forming a scale (reference float8_utils.py:19)

FP8_TYPES = {torch.float8_e4m3fn, torch.float8_e5m2, torch.float8_e4m3fnuz, torch.float8_e5m2fnuz}
_NATIVE_FP8 = (torch.float8_e4m3fn, torch.float8_e5m2)

if _config.use_fnuz_dtype:
    raise RuntimeError("fnuz float8 flavours are not supported: gfx950 uses the OCP e4m3fn / e5m2 formats")
e4m3_dtype = torch.float8_e4m3fn
e5m2_dtype = torch.float8_e5m2


def _check_fp8(float8_dtype) -> None:
    if float8_dtype not in FP8_TYPES:
        raise ValueError(f"Unsupported float8_dtype: {float8_dtype}")
    if float8_dtype not in _NATIVE_FP8:
        raise ValueError(f"Unsupported float8_dtype: {float8_dtype} (this build implements e4m3fn and e5m2)")


@torch.no_grad()
def amax_to_scale(amax: torch.Tensor, float8_dtype: torch.dtype, orig_dtype: torch.dtype) -> torch.Tensor:
    """fp8 scale of a (0-dim or stacked) amax tensor, fp32 (reference float8_utils.py:35-57).

    Evaluated with the same device operators, in amax's dtype, as the reference
    (``float / Tensor`` is ``reciprocal() * float``), so results are identical.  The
    single-tensor hot path does not come through here: ``tensor_to_scale`` fuses
    this arithmetic into the amax kernel.
    """
    _check_fp8(float8_dtype)
    _native._require_gpu(amax, "amax")
    res = torch.clamp(amax, min=EPS).reciprocal() * torch.finfo(float8_dtype).max
    if orig_dtype is torch.float16:
        res = torch.clamp(res, max=torch.finfo(torch.float16).max)
    return res.to(torch.float32)


@torch.no_grad()
def amax_history_to_scale(amax_history, float8_dtype, orig_dtype, history_to_scale_fn_type: Literal["max"]):
    """Scale from one amax history (reference float8_utils.py:60-77)."""
    if history_to_scale_fn_type != "max":
        raise NotImplementedError()
    return amax_to_scale(torch.max(amax_history), float8_dtype, orig_dtype)


@torch.no_grad()
def amax_history_to_scale_stack(amax_history, float8_dtype, orig_dtype, history_to_scale_fn_type: Literal["max"]):
    """Scales from a [n, history_len] stack of histories (reference float8_utils.py:80-99)."""
    if history_to_scale_fn_type != "max":
        raise NotImplementedError(
            f"Invalid history_to_scale_fn_type, only 'max' is supported. Got: {history_to_scale_fn_type}"
        )
    return amax_to_scale(torch.max(amax_history, dim=1).values, float8_dtype, orig_dtype)


@torch.no_grad()
def tensor_to_amax(x: torch.Tensor, reduce_amax: bool = False) -> torch.Tensor:
    """max|x| as a 0-dim tensor of x's dtype (reference float8_utils.py:102-112).

    ``reduce_amax`` asks for a MAX all-reduce over ranks; this build drives one GPU,
    so with an initialised process group of more than one rank it raises.
    """
    _no_multi_rank(reduce_amax)
    _native._require_gpu(x, "x")
    amax, _ = torch.ops.f8mi.amax_scale(x, e4m3_dtype, x.dtype, x.dtype == torch.float16)
    return amax.to(x.dtype)  # exact: the maximum is one of x's values


@torch.no_grad()
def tensor_to_scale(x: torch.Tensor, float8_dtype: torch.dtype, reduce_amax: bool = False) -> torch.Tensor:
    """Dynamic scale of x: one pass, amax and scale arithmetic in one kernel (reference :115-120)."""
    _check_fp8(float8_dtype)
    _no_multi_rank(reduce_amax)
    _native._require_gpu(x, "x")
    # through the custom op (one opaque node for torch.compile; the same launch in eager mode)
    _, scale = torch.ops.f8mi.amax_scale(x, float8_dtype, x.dtype, x.dtype == torch.float16)
    return scale


def to_fp8_saturated(x: torch.Tensor, float8_dtype: torch.dtype) -> torch.Tensor:
    """clamp to the fp8 range, then convert (reference float8_utils.py:123-139)."""
    _check_fp8(float8_dtype)
    _native._require_gpu(x, "x")
    one = torch.ones((), dtype=torch.float32, device=x.device)
    out, _ = torch.ops.f8mi.cast(x, one, float8_dtype, x.dtype, False)
    return out


def _no_multi_rank(reduce_amax: bool) -> None:
    if reduce_amax and torch.distributed.is_available() and torch.distributed.is_initialized():
        if torch.distributed.get_world_size() > 1:
            raise NotImplementedError("amax all-reduce across ranks: this build drives a single GPU")


def compute_error(x: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
    """Signal-to-quantisation-noise ratio of y against x, in dB (reference float8_utils.py:142-154)."""
    return 20 * torch.log10(torch.norm(x) / torch.norm(x - y))


def fp8_tensor_statistics(tensor, float8_dtype=e4m3_dtype) -> Tuple[int, ...]:
    """(#zeros, #entries at +-max) of a Float8Tensor's payload (reference float8_utils.py:157-176)."""
    if float8_dtype not in FP8_TYPES:
        raise ValueError(f"Unsupported float8_dtype: {float8_dtype}")
    hp = tensor._data.to(dtype=tensor._orig_dtype)
    top = torch.finfo(float8_dtype).max
    return ((hp == 0).sum().item(), (hp.abs() == top).sum().item())


def is_row_major(stride) -> bool:
    assert len(stride) == 2, "is_row_major only supports 2D tensors"
    return stride[0] > stride[1] and stride[1] == 1


def _get_min_alignment(size: int, alignment_value: int) -> int:
    """Smallest multiple of ``alignment_value`` that is >= ``size``."""
    return -(-size // alignment_value) * alignment_value


def pad_tensor_for_matmul(tensor: torch.Tensor, dims: Union[int, Iterable[int]]) -> torch.Tensor:
    """Zero-pads the chosen dims of a 2-D tensor up to multiples of 16 (reference :206-247).

    Kept for callers of the reference API; the GEMM kernel of this package needs no padding.
    """
    assert tensor.dim() == 2
    dims = (dims,) if isinstance(dims, int) else tuple(dims)
    rows, cols = tensor.shape
    new_rows = _get_min_alignment(rows, 16) if 0 in dims else rows
    new_cols = _get_min_alignment(cols, 16) if 1 in dims else cols
    if (new_rows, new_cols) == (rows, cols):
        return tensor
    if tensor.dtype in FP8_TYPES:  # F.pad has no fp8 kernels: pad the bytes (0x00 is +0)
        padded = torch.nn.functional.pad(tensor.view(torch.uint8), (0, new_cols - cols, 0, new_rows - rows))
        return padded.view(tensor.dtype)
    return torch.nn.functional.pad(tensor, (0, new_cols - cols, 0, new_rows - rows))
