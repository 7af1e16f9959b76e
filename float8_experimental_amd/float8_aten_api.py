"""The emulated float8 matmul as the aten-level op of the reference (mirror of ``float8_aten_api.py``).

Only reached when a layer is configured with ``emulate=True``: the operands are
dequantised elementwise and multiplied in fp32 with the device's ordinary
matmul.  It is an explicit option of the reference API, not a fallback: with
``emulate=False`` the matrix-core kernel is the only path.
"""
import torch
from torch.library import Library


def mm_float8_emulated(m1, s1, m2, s2, dtype3):
    """``mm(m1 / s1, m2 / s2)`` in fp32, result cast to ``dtype3`` (reference float8_aten_api.py:16-28)."""
    m1_fp32 = m1.float() / s1
    m2_fp32 = m2.float() / s2
    return torch.mm(m1_fp32, m2_fp32).to(dtype3)


def _mm_float8_emulated_meta(m1, s1, m2, s2, dtype3):
    return torch.empty((m1.shape[0], m2.shape[1]), dtype=dtype3, device=m1.device)


# ``torch.ops.aten.mm_float8_emulated`` (reference float8_aten_api.py:37-49).  The schema lives in the ``aten``
# namespace, which holds one definition per process: if the reference package was imported first, its definition
# (same schema, same arithmetic) is the one in place and nothing is added here.
if not hasattr(torch.ops.aten, "mm_float8_emulated"):
    lib = Library("aten", "FRAGMENT")
    lib.define("mm_float8_emulated(Tensor m1, Tensor s1, Tensor m2, Tensor s2, ScalarType dtype3) -> Tensor")
    lib.impl("mm_float8_emulated", mm_float8_emulated, "CUDA")
    lib.impl("mm_float8_emulated", _mm_float8_emulated_meta, "Meta")
