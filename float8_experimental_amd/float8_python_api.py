"""``addmm_float8_unwrapped``: the scaled fp8 matmul on plain tensors
(mirror of the reference's ``float8_python_api.py``, which forwards to ``torch._scaled_mm``).
"""
from typing import Optional

import torch

from . import _custom_ops  # noqa: F401  (registers torch.ops.f8mi.*)
from . import _native


def addmm_float8_unwrapped(a_data: torch.Tensor, a_scale: torch.Tensor, b_data: torch.Tensor, b_scale: torch.Tensor,
                           output_dtype: torch.dtype, output_scale: Optional[torch.Tensor] = None,
                           bias: Optional[torch.Tensor] = None, use_fast_accum: bool = False) -> torch.Tensor:
    """``(a_data @ b_data) / (a_scale * b_scale) (+ bias)`` on the gfx950 matrix cores.

    ``a_data`` is fp8 ``[m, k]``, ``b_data`` fp8 ``[k, n]``; as in the reference
    (float8_python_api.py:24-64) the scales are the tensors' forward scales and the
    kernel applies their reciprocals.  Any layout is taken: ``a_data`` row-major with
    ``b_data`` column-major (the pair ``torch._scaled_mm`` insists on) is read as it lies; a
    row-major ``b_data`` -- and a column-major ``a_data`` next to it -- is read transposed by the
    matrix-core kernel (f8mi_gemm_ex) where the product is large and aligned enough, and
    copied once where it is not.
    ``use_fast_accum`` has no effect on this hardware.  ``output_scale`` (fp8 output) is
    not implemented, as in the reference's own call sites, which always pass None.
    """
    if output_scale is not None:
        raise NotImplementedError("fp8 output of the scaled matmul is not supported")
    assert a_data.dim() == 2 and b_data.dim() == 2 and a_data.shape[1] == b_data.shape[0]
    _native._require_gpu(a_data, "a_data")
    return torch.ops.f8mi.scaled_mm(a_data, a_scale, b_data, b_scale, output_dtype, bias)
