"""The emulated float8 matmul (mirror of the reference's ``float8_aten_api.py``).

Only reached when a layer is configured with ``emulate=True``: the operands are
dequantised elementwise and multiplied in fp32 with the device's ordinary
matmul.  It is an explicit option of the reference API, not a fallback: with
``emulate=False`` the matrix-core kernel is the only path.
"""
import torch


def mm_float8_emulated(m1, s1, m2, s2, dtype3):
    """``mm(m1 / s1, m2 / s2)`` in fp32, result cast to ``dtype3`` (reference float8_aten_api.py:16-28)."""
    m1_fp32 = m1.float() / s1
    m2_fp32 = m2.float() / s2
    return torch.mm(m1_fp32, m2_fp32).to(dtype3)
